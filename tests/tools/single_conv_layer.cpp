// single_conv_layer - command-line harness for one convolution layer: the
// forward, backward-data and weight update passes.
//
// Test infrastructure: it runs the convolutions through the C++ poplin layer
// of this build (hence through the C ABI and the gfx950 kernels) and compares
// the results with the CPU oracle (oracle/conv_oracle.c), exactly as PopLibs'
// tools/single_conv_layer.cpp compares a device run with
// poplibs_test::conv::convolution / convolutionBackward / weightUpdate.  That
// tool's options are accepted under the same names
// (tools/single_conv_layer.cpp:171-430); the same data modes, comparison rule
// and exit codes apply:
//   * +-1 "Bernoulli" data with zero tolerance when the sums stay exactly
//     representable, else uniform random data with tolerances
//     (tools/single_conv_layer.cpp:941-1005, lib/poplibs_test/Util.cpp:167-196)
//   * element-wise checkIsClose (lib/poplibs_test/Util.cpp:198-217, 316-348)
//   * exit 0 = match, 1 = mismatch or bad usage, 77 = out of device memory
//     (tools/single_conv_layer.cpp:1531-1537).
// Options that only steer the IPU build of the graph (--tiles-per-ipu, --ipus,
// --input-load-width, --workers-per-tile, --remap-output-tensor,
// --enable-convolution-reuse, --report-var-storage, --profile, --profile-dir,
// the --test-planner-report-* family) are accepted and have no effect here.
// --test-planner compares the planner's estimate of every pass that ran with
// the time measured between two HIP events (reportPlanEstimatedCosts against
// the clock; tools/single_conv_layer.cpp:183, 857-888, 1490-1520 compare the
// IPU planner's estimates with a profile): the case fails when they differ
// by more than the factor --test-planner-tolerance (default 2.5) beyond 15 us
// of launch overhead.  --fwd-in-file / --fwd-out-file / --bwd-in-file /
// --bwd-out-file read and write a tensor in this harness's own container
// (magic "MXT1", element type, rank, dimensions, raw values in the external
// layout); Poplar's own binary tensor format is part of the closed SDK.
//
//   single_conv_layer --batch-file cases.json
// runs many invocations in one process (one HIP start-up for all):
// cases.json is [{"name": ..., "args": [...]}, ...]; every case prints
// "### CASE <name>", its output and "### RESULT <name> <exit code>".
#include "poplar/OptionFlags.hpp"
#include "poplar/exceptions.hpp"
#include "poplin/ConvParams.hpp"
#include "poplin/ConvUtil.hpp"
#include "poplin/ConvPreplan.hpp"
#include "poplin/Convolution.hpp"
#include "poputil/exceptions.hpp"

#include "../../poplibs_amd/src/Json.hpp"
#include "harness_util.hpp"

#include "mxconv.h"
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <map>
#include <random>
#include <set>
#include <sstream>
#include <string>
#include <vector>

extern "C" {
int oracle_convolution(
    unsigned, const unsigned *, const unsigned *, const unsigned *,
    const unsigned *, const unsigned *, const unsigned *,
    const unsigned char *, const unsigned *, const unsigned *,
    const unsigned *, const unsigned *, const unsigned *, const unsigned *,
    const unsigned char *, const unsigned *, const unsigned *,
    const unsigned *, const unsigned *, const unsigned *, unsigned, unsigned,
    unsigned, unsigned, const double *, const double *, const double *,
    double *, size_t, int);
int oracle_weight_update(
    unsigned num_field_dims, const unsigned *input_field_size,
    const unsigned *truncation_lower, const unsigned *truncation_upper,
    const unsigned *input_dilation, const unsigned *padding_lower,
    const unsigned *padding_upper, const unsigned char *flip_input,
    const unsigned *kernel_size, const unsigned *kernel_truncation_lower,
    const unsigned *kernel_truncation_upper, const unsigned *kernel_dilation,
    const unsigned *kernel_padding_lower, const unsigned *kernel_padding_upper,
    const unsigned char *flip_kernel, const unsigned *output_truncation_lower,
    const unsigned *output_truncation_upper, const unsigned *stride,
    const unsigned *output_padding_lower, const unsigned *output_padding_upper,
    unsigned batch_size, unsigned num_conv_groups, unsigned in_chans_per_group,
    unsigned out_chans_per_group, const double *activations,
    const double *deltas, double *weight_deltas, size_t weight_delta_elems,
    double *bias_deltas, int threads);
int oracle_convolution_backward(
    unsigned, const unsigned *, const unsigned *, const unsigned *,
    const unsigned *, const unsigned *, const unsigned *,
    const unsigned char *, const unsigned *, const unsigned *,
    const unsigned *, const unsigned *, const unsigned *, const unsigned *,
    const unsigned char *, const unsigned *, const unsigned *,
    const unsigned *, const unsigned *, const unsigned *, unsigned, unsigned,
    unsigned, unsigned, const double *, const double *, double *, size_t, int);
}

namespace {

using poplin::ConvParams;

struct UsageError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

[[noreturn]] void usage(const std::string &message) {
  throw UsageError(message);
}

/// "{1,2,3}" gives one value per dimension; a bare "2" is broadcast
/// (ShapeOption, include/poplibs_test/Util.hpp:262-394).
struct Shape {
  std::vector<long> values;
  bool broadcast = false;
};

Shape parseShape(const std::string &text) {
  Shape s;
  std::string t = text;
  if (!t.empty() && t.front() == '{') {
    if (t.back() != '}')
      usage("missing '}' in '" + text + "'");
    t = t.substr(1, t.size() - 2);
    std::stringstream ss(t);
    std::string item;
    while (std::getline(ss, item, ','))
      if (!item.empty())
        s.values.push_back(std::stol(item));
  } else {
    s.values.push_back(std::stol(t));
    s.broadcast = true;
  }
  return s;
}

template <class T> std::vector<T> expand(const Shape &s, size_t n, T dflt) {
  if (s.values.empty())
    return std::vector<T>(n, dflt);
  if (s.broadcast)
    return std::vector<T>(n, T(s.values[0]));
  if (s.values.size() != n)
    usage("option has " + std::to_string(s.values.size()) +
          " values for " + std::to_string(n) + " field dimensions");
  return std::vector<T>(s.values.begin(), s.values.end());
}

} // namespace

/// The harness's own tensor container: "MXT1", element type id (0 float,
/// 1 half, 2 quarter), rank, dimensions (uint64), then the raw values in the
/// external layout.
void saveTensor(const std::string &path, poplar::Type type,
                const std::vector<size_t> &shape,
                const std::vector<uint8_t> &bytes) {
  std::ofstream f(path, std::ios::binary);
  if (!f.good())
    throw poputil::poplibs_error("file " + path + " could not be opened");
  const uint32_t id = type == poplar::FLOAT ? 0 : type == poplar::HALF ? 1 : 2;
  const uint32_t rank = uint32_t(shape.size());
  f.write("MXT1", 4);
  f.write(reinterpret_cast<const char *>(&id), 4);
  f.write(reinterpret_cast<const char *>(&rank), 4);
  for (size_t d : shape) {
    const uint64_t v = d;
    f.write(reinterpret_cast<const char *>(&v), 8);
  }
  f.write(reinterpret_cast<const char *>(bytes.data()),
          std::streamsize(bytes.size()));
}

struct LoadedTensor {
  poplar::Type type = poplar::HALF;
  std::vector<size_t> shape;
  std::vector<uint8_t> bytes;
};

LoadedTensor loadTensor(const std::string &what, const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f.good())
    throw poputil::poplibs_error("<" + what + "> file " + path +
                                 " could not be opened");
  char magic[4];
  uint32_t id = 0, rank = 0;
  f.read(magic, 4);
  f.read(reinterpret_cast<char *>(&id), 4);
  f.read(reinterpret_cast<char *>(&rank), 4);
  if (!f.good() || std::memcmp(magic, "MXT1", 4) != 0 || id > 2 || rank > 8)
    throw poputil::poplibs_error("No Tensors in " + what);
  LoadedTensor t;
  t.type = id == 0 ? poplar::FLOAT : id == 1 ? poplar::HALF : poplar::QUARTER;
  size_t elems = 1;
  for (uint32_t d = 0; d != rank; ++d) {
    uint64_t v = 0;
    f.read(reinterpret_cast<char *>(&v), 8);
    t.shape.push_back(size_t(v));
    elems *= size_t(v);
  }
  t.bytes.resize(elems * t.type.size());
  f.read(reinterpret_cast<char *>(t.bytes.data()),
         std::streamsize(t.bytes.size()));
  if (!f.good() && !t.bytes.empty())
    throw poputil::poplibs_error("file " + path + " is truncated");
  return t;
}

std::string shapeText(const std::vector<size_t> &shape) {
  std::string s = "[";
  for (size_t i = 0; i != shape.size(); ++i)
    s += (i ? "," : "") + std::to_string(shape[i]);
  return s + "]";
}

std::string readFile(const std::string &path) {
  std::ifstream f(path);
  if (!f)
    usage("cannot read '" + path + "'");
  std::stringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

int runCase(int argc, char **argv) try {
  std::map<std::string, std::string> opt = parseCommandLine(argc, argv);
  static const char *known[] = {
      "help", "input-channels", "output-channels", "field", "kernel-size",
      "bias", "data-type", "input-type", "output-type", "fp8-scale-fwd",
      "fp8-scale-weights", "fp8-format-fwd", "fp8-format-weights",
      "truncation", "truncation-upper", "truncation-lower", "in-dilation",
      "padding", "padding-upper", "padding-lower", "flip-input",
      "kernel-truncation", "kernel-truncation-upper",
      "kernel-truncation-lower", "kernel-dilation", "kernel-padding",
      "kernel-padding-upper", "kernel-padding-lower", "flip-kernel",
      "output-truncation", "output-truncation-upper",
      "output-truncation-lower", "stride", "output-padding",
      "output-padding-upper", "output-padding-lower", "single-phase",
      "inference-only", "bwd-plan-constraints", "wu-plan-constraints",
      "plan-only", "inference-only", "tolerance", "absolute-tolerance",
      "batch-size", "conv-groups", "fwd-plan-constraints",
      "fwd-plan-constraints-file", "report-plan", "convolution-options",
      "preplan",
      "use-create-input", "num-determinism-checks", "ignore-data", "seed",
      "device-type", "profile", "timing-runs",
      "use-create-output", "fp8-scale-bwd", "fp8-format-bwd",
      "bwd-plan-constraints-file", "wu-plan-constraints-file", "fwd-in-file",
      "fwd-out-file", "bwd-in-file", "bwd-out-file", "test-planner",
      "test-planner-tolerance", "compile-only",
      // steer the IPU graph only: accepted, no effect
      "tiles-per-ipu", "ipus", "input-load-width", "workers-per-tile",
      "remap-output-tensor", "enable-convolution-reuse", "report-var-storage",
      "profile-dir", "test-planner-existing-profile",
      "test-planner-simulated-execution-file", "test-planner-report-all-tiles",
      "test-planner-report-all-serial-splits", "test-planner-report-verbose",
      "test-planner-print-vars"};
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
  for (const char *required : {"input-channels", "output-channels"})
    if (!has(required))
      usage(std::string("the option '--") + required + "' is required");
  // (tools/single_conv_layer.cpp:450-463)
  if (has("fwd-in-file") || has("bwd-in-file")) {
    if (has("fwd-in-file") &&
        (has("field") || has("input-type") || has("batch-size"))) {
      std::cerr << "Cannot specify --field, --batch-size or --input-type with "
                   "an input file\n";
      return 1;
    }
  }
  if (!has("field") && !has("fwd-in-file")) {
    std::cerr << "Must use an input file or specify --field\n";
    return 1;
  }
  // Passes (tools/single_conv_layer.cpp:715-735).
  const std::string phase = get("single-phase", "all");
  if (phase != "fwd" && phase != "bwd" && phase != "wu" && phase != "all")
    usage("--single-phase must be fwd, bwd, wu or all");
  const bool inferenceOnly = parseBool(get("inference-only", "false"));
  const bool doFwdPass = phase == "fwd" || phase == "all";
  const bool doBwdPass = !inferenceOnly && (phase == "bwd" || phase == "all");
  bool doWuPass = !inferenceOnly && (phase == "wu" || phase == "all");

  // ---- parameters (tools/single_conv_layer.cpp:768-790) -------------------
  poplar::Type inputType = parseType(get("data-type", "half"));
  poplar::Type outputType = inputType;
  if (has("input-type"))
    inputType = parseType(get("input-type"));
  if (has("output-type"))
    outputType = parseType(get("output-type"));
  size_t batchSize = std::stoul(get("batch-size", "1"));
  Shape field = has("field") ? parseShape(get("field")) : Shape{};
  // The forward input from a file: its type, batch size and field replace the
  // options' (tools/single_conv_layer.cpp:593-626).
  LoadedTensor fwdIn, bwdIn;
  if (has("fwd-in-file")) {
    fwdIn = loadTensor("fwd-in-file", get("fwd-in-file"));
    std::cout << "Importing FWD input from file, shape:"
              << shapeText(fwdIn.shape)
              << " Element type:" << fwdIn.type.toString() << "\n";
    if (fwdIn.shape.size() < 2)
      throw poputil::poplibs_error("No Tensors in fwd-in-file");
    if (!has("output-type") && outputType == inputType)
      outputType = fwdIn.type == poplar::QUARTER ? poplar::HALF : fwdIn.type;
    inputType = fwdIn.type;
    batchSize = fwdIn.shape[0];
    if (fwdIn.shape[1] != std::stoul(get("input-channels")) *
                              std::stoul(get("conv-groups", "1"))) {
      std::cerr << "The product of conv-groups and input-channels must be "
                   "equal to dimension 1 of the FWD input file tensor, which "
                   "is "
                << fwdIn.shape[1] << "\n";
      return 1;
    }
    field = Shape{};
    for (size_t d = 2; d != fwdIn.shape.size(); ++d)
      field.values.push_back(long(fwdIn.shape[d]));
  }
  // (a bare number is a one-dimensional field:
  // tools/single_conv_layer.cpp:653-654 takes the rank from the values given)
  field.broadcast = false;
  const size_t n = field.values.size();
  const auto fieldShape = expand<size_t>(field, n, 1);
  // (--kernel-size defaults to 1, tools/single_conv_layer.cpp:208-212)
  const auto kernelShape = expand<size_t>(
      has("kernel-size") ? parseShape(get("kernel-size")) : Shape{}, n, 1);
  auto both = [&](const char *base, const char *suffix) {
    const std::string specific = std::string(base) + suffix;
    return has(specific.c_str()) ? parseShape(opt[specific])
                                 : (has(base) ? parseShape(opt[base]) : Shape{});
  };
  auto flips = [&](const char *k) {
    const auto v = expand<long>(has(k) ? parseShape(opt[k]) : Shape{}, n, 0);
    return std::vector<bool>(v.begin(), v.end());
  };
  ConvParams::InputTransform inT(
      expand<unsigned>(both("truncation", "-lower"), n, 0),
      expand<unsigned>(both("truncation", "-upper"), n, 0),
      expand<unsigned>(has("in-dilation") ? parseShape(opt["in-dilation"])
                                          : Shape{},
                       n, 1),
      expand<unsigned>(both("padding", "-lower"), n, 0),
      expand<unsigned>(both("padding", "-upper"), n, 0), flips("flip-input"));
  ConvParams::InputTransform kT(
      expand<unsigned>(both("kernel-truncation", "-lower"), n, 0),
      expand<unsigned>(both("kernel-truncation", "-upper"), n, 0),
      expand<unsigned>(has("kernel-dilation")
                           ? parseShape(opt["kernel-dilation"])
                           : Shape{},
                       n, 1),
      expand<unsigned>(both("kernel-padding", "-lower"), n, 0),
      expand<unsigned>(both("kernel-padding", "-upper"), n, 0),
      flips("flip-kernel"));
  ConvParams::OutputTransform outT(
      expand<unsigned>(both("output-truncation", "-lower"), n, 0),
      expand<unsigned>(both("output-truncation", "-upper"), n, 0),
      expand<unsigned>(has("stride") ? parseShape(opt["stride"]) : Shape{}, n,
                       1),
      expand<unsigned>(both("output-padding", "-lower"), n, 0),
      expand<unsigned>(both("output-padding", "-upper"), n, 0));
  const ConvParams params(
      inputType, outputType, batchSize, fieldShape,
      kernelShape, std::stoul(get("input-channels")),
      std::stoul(get("output-channels")), std::stoul(get("conv-groups", "1")),
      inT, kT, outT);
  params.validate();
  if (doWuPass && inputType == poplar::QUARTER) {
    if (phase == "wu")
      throw poputil::poplibs_error(
          "the weight update pass takes half or float tensors");
    std::cout << "Weight update pass skipped: it takes half or float tensors\n";
    doWuPass = false;
  }

  // ---- options (tools/single_conv_layer.cpp:803-832) ----------------------
  poplar::OptionFlags options;
  options.set("pass", has("inference-only") ? "INFERENCE_FWD" : "TRAINING_FWD");
  // (a constraints string and a constraints file for one pass exclude each
  // other, tools/single_conv_layer.cpp:437-461)
  for (const char *pass : {"fwd", "bwd", "wu"}) {
    const std::string text = std::string(pass) + "-plan-constraints";
    if (has(text.c_str()) && has((text + "-file").c_str()) &&
        !get(text.c_str()).empty() && !get((text + "-file").c_str()).empty())
      throw poputil::poplibs_error("Both " + text + " and " + text +
                                   "-file were specified");
  }
  auto constraintsFor = [&](const char *pass) -> std::pair<bool, std::string> {
    const std::string text = std::string(pass) + "-plan-constraints";
    const std::string file = text + "-file";
    if (has(file.c_str()) && !get(file.c_str()).empty())
      return {true, readFile(get(file.c_str()))};
    if (has(text.c_str()))
      return {true, get(text.c_str())};
    return {false, ""};
  };
  const auto fwdConstraints = constraintsFor("fwd");
  if (fwdConstraints.first)
    options.set("planConstraints", fwdConstraints.second);
  if (has("remap-output-tensor"))
    options.set("remapOutputTensor",
                parseBool(get("remap-output-tensor")) ? "true" : "false");
  if (has("convolution-options")) {
    const auto doc = poplibs_amd::json::parse(get("convolution-options"));
    if (!doc.isObject())
      usage("--convolution-options must be a JSON object");
    for (const auto &m : doc.members)
      options.set(m.first, m.second.text);
  }
  poplin::convolutionValidateOptions(options);

  // Backward pass = forward convolution of the output gradient with the
  // gradient parameters and transposed, flipped weights
  // (tools/single_conv_layer.cpp:793, 1064-1082).
  const ConvParams bwdParams = poplin::getGradientParams(params);
  poplar::OptionFlags bwdOptions = options;
  const auto bwdConstraints = constraintsFor("bwd");
  if (bwdConstraints.first)
    bwdOptions.set("planConstraints", bwdConstraints.second);
  else if (fwdConstraints.first)
    bwdOptions.set("planConstraints", "");
  poplin::convolutionValidateOptions(bwdOptions);
  // Weight update: the forward options with pass TRAINING_WU
  // (tools/single_conv_layer.cpp:821-824).
  poplar::OptionFlags wuOptions = options;
  wuOptions.set("pass", "TRAINING_WU");
  const auto wuConstraints = constraintsFor("wu");
  if (wuConstraints.first)
    wuOptions.set("planConstraints", wuConstraints.second);
  else if (fwdConstraints.first)
    wuOptions.set("planConstraints", "");
  poplin::convolutionValidateOptions(wuOptions);
  const auto flops = poplin::getFwdFlops(params);
  poplin::PlanningCache cache;
  // Plan the passes that run ahead of their use
  // (tools/single_conv_layer.cpp:415-417, 831-850).
  if (parseBool(get("preplan", "true"))) {
    std::set<poplin::ConvPlanParams> convs;
    if (doFwdPass)
      convs.insert(std::make_tuple(nullptr, params, &options));
    if (doBwdPass)
      convs.insert(std::make_tuple(nullptr, bwdParams, &bwdOptions));
    if (doWuPass)
      convs.insert(std::make_tuple(
          nullptr, poplin::getWeightUpdateParams(params), &wuOptions));
    poplin::preplan(convs, {}, cache);
  }
  const bool reportPlan = parseBool(get("report-plan", "false")) || has("plan-only");
  auto reportCosts = [&](const ConvParams &p, const poplar::OptionFlags &o) {
    const poplin::PlanCosts costs =
        poplin::reportPlanEstimatedCosts(p, o, &cache);
    std::cout << "  estimated cycles: ";
    if (costs.cycles == poplin::PlanCosts::unknown)
      std::cout << "unknown";
    else
      std::cout << costs.cycles;
    std::cout << ", temporary memory: " << costs.memory << " bytes\n";
  };
  if (doFwdPass) {
    std::cout << "Forward FLOPs: " << flops << "\n";
    if (reportPlan) {
      std::cout << "Forward plan:\n";
      poplin::reportPlanInfo(std::cout, params, options, &cache);
      reportCosts(params, options);
    }
  }
  if (doBwdPass) {
    std::cout << "Backward FLOPs: " << poplin::getFwdFlops(bwdParams) << "\n";
    if (reportPlan) {
      std::cout << "Backward plan:\n";
      poplin::reportPlanInfo(std::cout, bwdParams, bwdOptions, &cache);
      reportCosts(bwdParams, bwdOptions);
    }
  }
  if (doWuPass) {
    std::cout << "WU FLOPs: " << poplin::getWuFlops(params) << "\n";
    if (reportPlan) {
      std::cout << "WU plan:\n";
      poplin::reportWeightUpdatePlanInfo(std::cout, params, wuOptions, &cache);
    }
  }
  if (has("plan-only") || has("compile-only"))
    return 0;

  // ---- data (tools/single_conv_layer.cpp:941-1005, 1183-1213) -------------
  const auto outField = params.getOutputFieldShape();
  size_t inElems = params.batchSize * params.getNumInputChans();
  size_t wElems = params.numConvGroups * params.outputChannelsPerConvGroup *
                  params.inputChannelsPerConvGroup;
  size_t outElems = params.batchSize * params.getNumOutputChans();
  for (size_t d = 0; d != n; ++d) {
    inElems *= fieldShape[d];
    wElems *= kernelShape[d];
    outElems *= outField[d];
  }
  const bool useBias = parseBool(get("bias", "true"));
  double relTol = has("tolerance") ? std::stod(get("tolerance"))
                                   : (outputType == poplar::FLOAT ? 0.01 : 0.1);
  double absTol = has("absolute-tolerance")
                      ? std::stod(get("absolute-tolerance"))
                      : (outputType == poplar::FLOAT ? 1e-6 : 1e-5);
  const unsigned determinismChecks =
      unsigned(std::stoul(get("num-determinism-checks", "0")));
  // The longest sum any pass forms (tools/single_conv_layer.cpp:941-975).
  size_t macsPerOut = outElems ? (flops / 2) / outElems : 0;
  if (doBwdPass && inElems)
    macsPerOut = std::max<size_t>(macsPerOut, (flops / 2) / inElems);
  if (doWuPass && wElems)
    macsPerOut = std::max<size_t>(macsPerOut, (flops / 2) / wElems);
  const size_t maxInt = std::min(maxContiguousInteger(inputType),
                                 maxContiguousInteger(outputType));
  const bool uniformData = determinismChecks || macsPerOut > 10 * maxInt;
  if (uniformData) {
    std::cout << "Using uniform random data\n";
  } else {
    std::cout << "Using random binary {-1,1} data with no error tolerance\n";
    if (!has("tolerance"))
      relTol = 0;
    if (!has("absolute-tolerance"))
      absTol = 0;
  }
  poplin::QuarterMetadata inMeta, wMeta;
  auto fmt = [&](const char *k) {
    const std::string f = get(k, "quart143");
    if (f != "quart143" && f != "quart152")
      usage(std::string("--") + k + " must be quart143 or quart152");
    return f == "quart143" ? poplin::QuarterMetadata::Format::F143
                           : poplin::QuarterMetadata::Format::F152;
  };
  inMeta.format = fmt("fp8-format-fwd");
  wMeta.format = fmt("fp8-format-weights");
  inMeta.scale = std::stoi(get("fp8-scale-fwd", "1"));
  wMeta.scale = std::stoi(get("fp8-scale-weights", "2"));
  // the backward pass's input, the gradient of the forward output
  // (tools/single_conv_layer.cpp:155-158: quart143, scale 1 by default)
  poplin::QuarterMetadata zMeta;
  zMeta.format = fmt("fp8-format-bwd");
  zMeta.scale = std::stoi(get("fp8-scale-bwd", "1"));

  std::mt19937 rng(unsigned(std::stoul(get("seed", "5489"))));
  auto fill = [&](std::vector<double> &v, poplar::Type type, double lo,
                  double hi) {
    if (type == poplar::QUARTER) {
      // small integers, exactly representable (lib/poplibs_test/Util.cpp:
      // 54-56, 140-142); scaled so that the metadata scale leaves them exact
      std::uniform_int_distribution<int> d(uniformData ? int(lo) : -1,
                                           uniformData ? int(hi) : 1);
      for (auto &x : v)
        x = d(rng);
    } else if (uniformData) {
      std::uniform_real_distribution<double> d(lo, hi);
      for (auto &x : v)
        x = d(rng);
    } else {
      std::bernoulli_distribution d;
      for (auto &x : v)
        x = d(rng) ? 1.0 : -1.0;
    }
  };
  std::vector<double> acts(inElems), weights(wElems),
      biases(params.getNumOutputChans(), 0.0), zDeltas(outElems);
  fill(acts, inputType, -2, 2);
  fill(weights, inputType, -1, 1);
  fill(zDeltas, inputType, -3, 3);
  if (useBias)
    fill(biases, outputType == poplar::QUARTER ? poplar::HALF : outputType,
         uniformData ? -2 : -1, uniformData ? 6 : 1);
  if (inputType == poplar::QUARTER) {
    // keep the stored integers exact under the metadata scale
    for (auto &x : acts)
      x = std::ldexp(x, inMeta.scale);
    for (auto &x : weights)
      x = std::ldexp(x, wMeta.scale);
    for (auto &x : zDeltas)
      x = std::ldexp(x, zMeta.scale);
  }
  if (has("fwd-in-file")) {
    // (the file's values as they are; quarter values under --fp8-scale-fwd)
    if (fwdIn.bytes.size() != inElems * inputType.size())
      throw poputil::poplibs_error("fwd-in-file does not hold the input");
    if (inputType == poplar::QUARTER) {
      for (size_t i = 0; i != inElems; ++i)
        acts[i] = std::ldexp(
            oracle_fp8_decode(fwdIn.bytes[i], int(inMeta.format)),
            inMeta.scale);
    } else {
      acts = decode(fwdIn.bytes, inputType);
    }
  }
  if (has("bwd-in-file")) {
    bwdIn = loadTensor("bwd-in-file", get("bwd-in-file"));
    std::cout << "Importing BWD input from file, shape:"
              << shapeText(bwdIn.shape)
              << " Element type:" << bwdIn.type.toString() << "\n";
    if (bwdIn.type != inputType ||
        bwdIn.bytes.size() != outElems * inputType.size())
      throw poputil::poplibs_error(
          "bwd-in-file does not hold the gradient of the forward output");
    if (inputType == poplar::QUARTER) {
      for (size_t i = 0; i != outElems; ++i)
        zDeltas[i] = std::ldexp(
            oracle_fp8_decode(bwdIn.bytes[i], int(zMeta.format)), zMeta.scale);
    } else {
      zDeltas = decode(bwdIn.bytes, inputType);
    }
  }
  const auto actBytes = encode(acts, inputType, inMeta);
  const auto weightBytes = encode(weights, inputType, wMeta);
  const auto biasBytes = encode(biases, outputType, {});
  const auto zDeltaBytes = encode(zDeltas, inputType, zMeta);

  // ---- device run ----------------------------------------------------------
  poplin::Stream prog;
  // --test-planner: per pass, the planner's estimate against the time
  // between two HIP events around 20 calls (after 3 untimed ones).
  struct PlannerCheck {
    std::string pass;
    double estimateUs, measuredUs;
  };
  std::vector<PlannerCheck> plannerChecks;
  const bool testPlanner = has("test-planner");
  auto measure = [&](const std::string &pass, const ConvParams &p,
                     const poplar::OptionFlags &o, auto &&call) {
    if (!testPlanner)
      return;
    const poplin::PlanCosts costs =
        poplin::reportPlanEstimatedCosts(p, o, &cache);
    for (int i = 0; i != 3; ++i)
      call();
    prog.synchronize();
    hipEvent_t start, stop;
    if (hipEventCreate(&start) != hipSuccess ||
        hipEventCreate(&stop) != hipSuccess)
      throw poputil::poplibs_error("hipEventCreate failed");
    const hipStream_t stream = static_cast<hipStream_t>(prog.handle());
    const int reps = 20;
    (void)hipEventRecord(start, stream);
    for (int i = 0; i != reps; ++i)
      call();
    (void)hipEventRecord(stop, stream);
    (void)hipEventSynchronize(stop);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, start, stop);
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    plannerChecks.push_back(
        {pass,
         costs.cycles == poplin::PlanCosts::unknown
             ? -1.0
             : double(costs.cycles) / poplin::PlanCosts::clockMHz,
         double(ms) * 1e3 / reps});
  };
  // --use-create-input=false: an input in the plan-independent external
  // layout [B][C][field...], which the convolution rearranges itself
  // (tools/single_conv_layer.cpp:399-406, 1009-1020).
  const bool useCreateInput = parseBool(get("use-create-input", "true"));
  poplin::DeviceTensor in;
  if (useCreateInput) {
    in = poplin::createInput(params, options, &cache);
  } else {
    std::vector<size_t> shape{params.batchSize, params.getNumInputChans()};
    shape.insert(shape.end(), fieldShape.begin(), fieldShape.end());
    in = poplin::DeviceTensor(inputType, shape,
                              poplin::DeviceTensor::Layout::External,
                              std::max<size_t>(inElems * inputType.size(), 1));
  }
  auto w = poplin::createWeights(params, options, &cache);
  in.metadata = inMeta;
  w.metadata = wMeta;
  std::vector<uint8_t> result(outElems * outputType.size());
  std::vector<uint8_t> first;
  const bool ignoreData = has("ignore-data");
  const unsigned runs = doFwdPass ? 1 + determinismChecks : 0;
  for (unsigned run = 0; run != runs; ++run) {
    if (!ignoreData) {
      if (useCreateInput)
        poplin::writeTensor(in, actBytes.data(), prog, params, options, &cache);
      else
        poplin::writeTensor(in, actBytes.data(), prog);
      poplin::writeTensor(w, weightBytes.data(), prog, params, options, &cache);
    }
    poplin::DeviceTensor out;
    if (parseBool(get("use-create-output", "false"))) {
      // (tools/single_conv_layer.cpp:407, 1027-1035)
      out = poplin::createConvOutput(params, options, &cache);
      poplin::convolutionWithOutput(in, w, out, params, false, prog, options,
                                    &cache);
    } else {
      out = poplin::convolution(in, w, params, false, prog, options, &cache);
    }
    if (useBias) {
      auto b = poplin::createBiases(out);
      if (!ignoreData)
        poplin::writeTensor(b, biasBytes.data(), prog, params, options, &cache);
      poplin::addBias(out, b, prog);
      prog.synchronize();
    }
    if (!ignoreData)
      poplin::readTensor(out, result.data(), prog, params, options, &cache);
    prog.synchronize();
    if (run == 0)
      first = result;
    else if (result != first) {
      std::cerr << "Determinism check " << run
                << " failed: results differ between runs\n";
      return 1;
    }
  }
  if (doFwdPass && testPlanner) {
    auto out = poplin::createConvOutput(params, options, &cache);
    measure("fwd", params, options, [&] {
      poplin::convolutionWithOutput(in, w, out, params, false, prog, options,
                                    &cache);
    });
  }
  if (has("fwd-out-file") && doFwdPass && !has("ignore-data")) {
    std::vector<size_t> shape{params.batchSize, params.getNumOutputChans()};
    shape.insert(shape.end(), outField.begin(), outField.end());
    std::cout << "Saving FWD tensor with shape:" << shapeText(shape)
              << " Element type:" << outputType.toString() << "\n";
    saveTensor(get("fwd-out-file"), outputType, shape, result);
  }
  // Backward pass: the forward weights, in the external layout, go in with
  // transposeAndFlipWeights = true.
  std::vector<uint8_t> bwdResult(inElems * outputType.size());
  if (doBwdPass) {
    std::vector<size_t> wShape{params.numConvGroups,
                               params.outputChannelsPerConvGroup,
                               params.inputChannelsPerConvGroup};
    wShape.insert(wShape.end(), kernelShape.begin(), kernelShape.end());
    poplin::DeviceTensor fwdWeights(inputType, wShape,
                                    poplin::DeviceTensor::Layout::External,
                                    std::max<size_t>(weightBytes.size(), 1));
    fwdWeights.metadata = wMeta;
    auto deltas = poplin::createInput(bwdParams, bwdOptions, &cache);
    deltas.metadata = zMeta;
    if (!ignoreData) {
      poplin::writeTensor(fwdWeights, weightBytes.data(), prog, params, options,
                          &cache);
      poplin::writeTensor(deltas, zDeltaBytes.data(), prog, bwdParams,
                          bwdOptions, &cache);
    }
    auto prevDeltas = poplin::convolution(deltas, fwdWeights, bwdParams, true,
                                          prog, bwdOptions, &cache);
    if (!ignoreData)
      poplin::readTensor(prevDeltas, bwdResult.data(), prog, bwdParams,
                         bwdOptions, &cache);
    prog.synchronize();
    if (testPlanner) {
      // (the estimate covers the convolution: the weights are turned round
      // once, outside the timed calls)
      std::vector<size_t> flippedShape = wShape;
      std::swap(flippedShape[1], flippedShape[2]);
      poplin::DeviceTensor flipped(inputType, flippedShape,
                                   poplin::DeviceTensor::Layout::External,
                                   std::max<size_t>(weightBytes.size(), 1));
      flipped.metadata = wMeta;
      poplin::weightsTransposeChansFlipXY(fwdWeights, flipped, prog);
      std::vector<uint8_t> flippedBytes(weightBytes.size());
      poplin::readTensor(flipped, flippedBytes.data(), prog);
      auto packed = poplin::createWeights(bwdParams, bwdOptions, &cache);
      packed.metadata = wMeta;
      poplin::writeTensor(packed, flippedBytes.data(), prog, bwdParams,
                          bwdOptions, &cache);
      auto out = poplin::createConvOutput(bwdParams, bwdOptions, &cache);
      measure("bwd", bwdParams, bwdOptions, [&] {
        poplin::convolutionWithOutput(deltas, packed, out, bwdParams, false,
                                      prog, bwdOptions, &cache);
      });
    }
    if (has("bwd-out-file") && !ignoreData) {
      std::vector<size_t> shape{params.batchSize, params.getNumInputChans()};
      shape.insert(shape.end(), fieldShape.begin(), fieldShape.end());
      std::cout << "Saving BWD tensor with shape:" << shapeText(shape)
                << " Element type:" << outputType.toString() << "\n";
      saveTensor(get("bwd-out-file"), outputType, shape, bwdResult);
    }
  }
  // Weight update: weights += -learningRate * deltas on a copy of the
  // weights in the external layout, biases likewise
  // (tools/single_conv_layer.cpp:1056-1094).
  const double learningRate = uniformData ? 0.05 : 1.0;
  std::vector<uint8_t> wuWeights(weightBytes.size()),
      wuBiases(biasBytes.size());
  if (doWuPass) {
    std::vector<size_t> wShape{params.numConvGroups,
                               params.outputChannelsPerConvGroup,
                               params.inputChannelsPerConvGroup};
    wShape.insert(wShape.end(), kernelShape.begin(), kernelShape.end());
    poplin::DeviceTensor master(inputType, wShape,
                                poplin::DeviceTensor::Layout::External,
                                std::max<size_t>(weightBytes.size(), 1));
    // The deltas are held the way a convolution leaves its output and the
    // backward pass takes its input, whose shape and type they have.
    auto zIn = poplin::createInput(bwdParams, bwdOptions, &cache);
    if (!ignoreData) {
      poplin::writeTensor(master, weightBytes.data(), prog);
      poplin::writeTensor(zIn, zDeltaBytes.data(), prog, bwdParams, bwdOptions,
                          &cache);
      if (useCreateInput)
        poplin::writeTensor(in, actBytes.data(), prog, params, options, &cache);
      else
        poplin::writeTensor(in, actBytes.data(), prog);
    }
    poplin::convolutionWeightUpdate(zIn, master, in, params,
                                    float(-learningRate), prog, wuOptions,
                                    &cache);
    if (useBias) {
      poplin::DeviceTensor b(outputType, {params.getNumOutputChans()},
                             poplin::DeviceTensor::Layout::External,
                             std::max<size_t>(biasBytes.size(), 1));
      if (!ignoreData)
        poplin::writeTensor(b, biasBytes.data(), prog);
      poplin::convolutionBiasUpdate(zIn, b, float(-learningRate), options,
                                    prog);
      if (!ignoreData)
        poplin::readTensor(b, wuBiases.data(), prog);
    }
    if (!ignoreData)
      poplin::readTensor(master, wuWeights.data(), prog);
    prog.synchronize();
    if (testPlanner) {
      // The estimate covers the pass's kernels: they are timed through the C
      // ABI on tensors already in the device layouts, without the C++
      // layer's allocations and conversions around them.
      std::vector<const char *> keys, values;
      for (const auto &kv : wuOptions) {
        keys.push_back(kv.first.c_str());
        values.push_back(kv.second.c_str());
      }
      mxconv_params c;
      params.toC(c);
      mxconv_plan *wuPlan = nullptr;
      size_t wsBytes = 0;
      if (mxconv_weight_update_plan_create(&c, keys.data(), values.data(),
                                           keys.size(), &wuPlan) != MXCONV_OK ||
          mxconv_weight_update_workspace_bytes(wuPlan, &wsBytes) != MXCONV_OK)
        throw poputil::poplibs_error(mxconv_last_error());
      auto actsCl = poplin::createInput(params, options, &cache);
      if (!ignoreData)
        poplin::writeTensor(actsCl, actBytes.data(), prog, params, options,
                            &cache);
      poplin::DeviceTensor deltasOut(
          inputType, wShape, poplin::DeviceTensor::Layout::External,
          std::max<size_t>(weightBytes.size(), 1));
      poplin::DeviceTensor ws(poplar::FLOAT, {wsBytes / 4 + 1},
                              poplin::DeviceTensor::Layout::External,
                              wsBytes + 4);
      measure("wu", poplin::getWeightUpdateParams(params), wuOptions, [&] {
        if (mxconv_calculate_weight_deltas(
                wuPlan, zIn.data(), actsCl.data(), deltasOut.data(), ws.data(),
                wsBytes,
                reinterpret_cast<mxconv_stream>(prog.handle())) != MXCONV_OK)
          throw poputil::poplibs_error(mxconv_last_error());
      });
      mxconv_plan_destroy(wuPlan);
    }
  }
  if (has("timing-runs") && doFwdPass) {
    const unsigned reps = unsigned(std::stoul(get("timing-runs")));
    auto out = poplin::createConvOutput(params, options, &cache);
    poplin::convolutionWithOutput(in, w, out, params, false, prog, options,
                                  &cache);
    prog.synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    for (unsigned i = 0; i != reps; ++i)
      poplin::convolutionWithOutput(in, w, out, params, false, prog, options,
                                    &cache);
    prog.synchronize();
    const double s =
        std::chrono::duration<double>(std::chrono::steady_clock::now() - t0)
            .count() /
        reps;
    std::cout << "Forward time per call: " << s * 1e6 << " us, "
              << flops / s / 1e12 << " TFLOP/s\n";
  }
  bool plannerOk = true;
  if (testPlanner) {
    const double tol = std::stod(get("test-planner-tolerance", "2.5"));
    std::cout << "Planner estimates against measurements (factor " << tol
              << " beyond 15 us of launch overhead allowed):\n";
    for (const auto &c : plannerChecks) {
      std::cout << "  " << c.pass << ": estimated ";
      if (c.estimateUs < 0) {
        std::cout << "unknown (the cost model does not cover this kernel), "
                     "measured "
                  << c.measuredUs << " us\n";
        continue;
      }
      const bool ok = c.measuredUs <= tol * c.estimateUs + 15.0 &&
                      c.estimateUs <= tol * c.measuredUs + 15.0;
      std::cout << c.estimateUs << " us, measured " << c.measuredUs
                << " us per call" << (ok ? "" : "  <-- beyond the tolerance")
                << "\n";
      plannerOk = plannerOk && ok;
    }
  }
  if (ignoreData) {
    std::cout << "Results not checked (--ignore-data)\n";
    return plannerOk ? 0 : 1;
  }

  // ---- host model and comparison (tools/single_conv_layer.cpp:1239-1252,
  // 1362-1368) ---------------------------------------------------------------
  auto u = [&](const std::vector<unsigned> &v) { return v; };
  auto shapeU = [](const std::vector<size_t> &v) {
    return std::vector<unsigned>(v.begin(), v.end());
  };
  auto flagsU = [](const std::vector<bool> &v) {
    return std::vector<unsigned char>(v.begin(), v.end());
  };
  // one spare element so that rank-0 fields still have storage to point at
  auto pad = [](std::vector<unsigned> v) {
    v.push_back(0);
    return v;
  };
  const auto fs = pad(shapeU(fieldShape)), ks = pad(shapeU(kernelShape));
  const auto itl = pad(u(inT.truncationLower)), itu = pad(u(inT.truncationUpper)),
             idl = pad(u(inT.dilation)), ipl = pad(u(inT.paddingLower)),
             ipu = pad(u(inT.paddingUpper));
  const auto ktl = pad(u(kT.truncationLower)), ktu = pad(u(kT.truncationUpper)),
             kdl = pad(u(kT.dilation)), kpl = pad(u(kT.paddingLower)),
             kpu = pad(u(kT.paddingUpper));
  const auto otl = pad(u(outT.truncationLower)),
             otu = pad(u(outT.truncationUpper)), ost = pad(u(outT.stride)),
             opl = pad(u(outT.paddingLower)), opu = pad(u(outT.paddingUpper));
  auto fi = flagsU(inT.flip), fk = flagsU(kT.flip);
  fi.push_back(0);
  fk.push_back(0);
  acts.push_back(0);
  weights.push_back(0);
  zDeltas.push_back(0);
  // checkIsClose element by element, plus the relative L2 error.
  auto compare = [&](const char *name, const std::vector<uint8_t> &bytes,
                     std::vector<double> &expected, size_t count,
                     poplar::Type type) {
    expected.resize(count);
    // The host model's result is rounded to the tensor's type before
    // comparing, as the reference does when it copies the model output into
    // a typed buffer.
    encode(expected, type, {});
    const auto actual = decode(bytes, type);
    unsigned mismatches = 0;
    double num = 0, den = 0;
    for (size_t i = 0; i != count; ++i) {
      const double a = actual[i], e = expected[i];
      num += (a - e) * (a - e);
      den += e * e;
      const bool bothNan = std::isnan(a) && std::isnan(e);
      if ((!bothNan && (std::isnan(a) || std::isnan(e))) ||
          (!isClose(a, e, relTol) && std::fabs(e - a) > absTol)) {
        if (mismatches++ < 20)
          std::cerr << "mismatch on element " << name << "[" << i
                    << "]: expected=" << e << " actual=" << a
                    << " (abs=" << a - e << ", rel=" << (a / e - 1.0) * 100.0
                    << "%)\n";
      }
    }
    std::cout << "Relative L2 error vs host model (" << name
              << "): " << (den > 0 ? std::sqrt(num / den) : std::sqrt(num))
              << "\n";
    if (mismatches)
      std::cerr << name << " validation failed (" << mismatches
                << " mismatches)\n";
    return mismatches == 0;
  };
  bool ok = true;
  if (doFwdPass) {
    std::vector<double> expected(outElems + 1);
    const int rc = oracle_convolution(
        unsigned(n), fs.data(), itl.data(), itu.data(), idl.data(), ipl.data(),
        ipu.data(), fi.data(), ks.data(), ktl.data(), ktu.data(), kdl.data(),
        kpl.data(), kpu.data(), fk.data(), otl.data(), otu.data(), ost.data(),
        opl.data(), opu.data(), unsigned(params.batchSize),
        unsigned(params.numConvGroups),
        unsigned(params.inputChannelsPerConvGroup),
        unsigned(params.outputChannelsPerConvGroup), acts.data(),
        weights.data(), biases.data(), expected.data(), outElems, 8);
    if (rc != 0) {
      std::cerr << "host model failed with code " << rc << "\n";
      return 1;
    }
    ok = compare("fwd", result, expected, outElems, outputType) && ok;
  }
  if (doBwdPass) {
    std::vector<double> expected(inElems + 1);
    const int rc = oracle_convolution_backward(
        unsigned(n), fs.data(), itl.data(), itu.data(), idl.data(), ipl.data(),
        ipu.data(), fi.data(), ks.data(), ktl.data(), ktu.data(), kdl.data(),
        kpl.data(), kpu.data(), fk.data(), otl.data(), otu.data(), ost.data(),
        opl.data(), opu.data(), unsigned(params.batchSize),
        unsigned(params.numConvGroups),
        unsigned(params.inputChannelsPerConvGroup),
        unsigned(params.outputChannelsPerConvGroup), zDeltas.data(),
        weights.data(), expected.data(), inElems, 8);
    if (rc != 0) {
      std::cerr << "host model (backward) failed with code " << rc << "\n";
      return 1;
    }
    ok = compare("bwd", bwdResult, expected, inElems, outputType) && ok;
  }
  if (doWuPass) {
    // tools/single_conv_layer.cpp:1270-1281, 1410-1436
    std::vector<double> weightDeltas(wElems + 1),
        biasDeltas(params.getNumOutputChans() + 1);
    const int rc = oracle_weight_update(
        unsigned(n), fs.data(), itl.data(), itu.data(), idl.data(), ipl.data(),
        ipu.data(), fi.data(), ks.data(), ktl.data(), ktu.data(), kdl.data(),
        kpl.data(), kpu.data(), fk.data(), otl.data(), otu.data(), ost.data(),
        opl.data(), opu.data(), unsigned(params.batchSize),
        unsigned(params.numConvGroups),
        unsigned(params.inputChannelsPerConvGroup),
        unsigned(params.outputChannelsPerConvGroup), acts.data(),
        zDeltas.data(), weightDeltas.data(), wElems, biasDeltas.data(), 8);
    if (rc != 0) {
      std::cerr << "host model (weight update) failed with code " << rc << "\n";
      return 1;
    }
    std::vector<double> modelWeights(wElems);
    for (size_t i = 0; i != wElems; ++i)
      modelWeights[i] = weights[i] + learningRate * -weightDeltas[i];
    ok = compare("weights", wuWeights, modelWeights, wElems, inputType) && ok;
    if (useBias) {
      std::vector<double> modelBiases(params.getNumOutputChans());
      for (size_t i = 0; i != modelBiases.size(); ++i)
        modelBiases[i] = biases[i] + learningRate * -biasDeltas[i];
      ok = compare("biases", wuBiases, modelBiases, modelBiases.size(),
                   outputType) && ok;
    }
  }
  if (!ok)
    return 1;
  std::cout << "Validation passed\n";
  if (!plannerOk) {
    std::cerr << "planner estimates beyond the tolerance\n";
    return 1;
  }
  return 0;
} catch (const UsageError &e) {
  std::cerr << "error: " << e.what() << "\n"
            << "usage: single_conv_layer --input-channels N --output-channels "
               "N --field {H,W} [--kernel-size {h,w}] [options]\n"
               "  see the header of tests/tools/single_conv_layer.cpp for the "
               "option list\n";
  return 1;
} catch (const poplar::graph_memory_allocation_error &e) {
  std::cerr << e.what() << std::endl;
  return 77;
} catch (const std::exception &e) {
  std::cerr << "error: " << e.what() << std::endl;
  return 1;
}

int main(int argc, char **argv) {
  if (argc == 3 && std::string(argv[1]) == "--batch-file") {
    // many invocations, one process; everything goes to stdout
    std::cerr.rdbuf(std::cout.rdbuf());
    poplibs_amd::json::Value doc;
    try {
      doc = poplibs_amd::json::parse(readFile(argv[2]));
    } catch (const std::exception &e) {
      std::cout << "error: " << e.what() << "\n";
      return 1;
    }
    int failed = 0;
    for (const auto &test : doc.items) {
      std::string name;
      std::vector<std::string> args{"single_conv_layer"};
      for (const auto &m : test.members) {
        if (m.first == "name")
          name = m.second.text;
        if (m.first == "args")
          for (const auto &a : m.second.items)
            args.push_back(a.text);
      }
      std::vector<char *> av;
      for (auto &a : args)
        av.push_back(const_cast<char *>(a.c_str()));
      std::cout << "### CASE " << name << std::endl;
      const int rc = runCase(int(av.size()), av.data());
      std::cout << "### RESULT " << name << " " << rc << std::endl;
      failed += rc != 0;
    }
    return failed ? 1 : 0;
  }
  return runCase(argc, argv);
}
