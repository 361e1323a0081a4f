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
#include "poplar/OptionFlags.hpp"
#include "poplar/exceptions.hpp"
#include "poplin/ConvParams.hpp"
#include "poplin/ConvUtil.hpp"
#include "poplin/ConvPreplan.hpp"
#include "poplin/Convolution.hpp"
#include "poputil/exceptions.hpp"

#include "../../poplibs_amd/src/Json.hpp"
#include "harness_util.hpp"

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

[[noreturn]] void usage(const std::string &message) {
  std::cerr << "error: " << message << "\n"
            << "usage: single_conv_layer --input-channels N --output-channels "
               "N --field {H,W} --kernel-size {h,w} [options]\n"
               "  see the header of tests/tools/single_conv_layer.cpp for the "
               "option list\n";
  std::exit(1);
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

int main(int argc, char **argv) try {
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
      "device-type", "profile", "timing-runs"};
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
  for (const char *required :
       {"input-channels", "output-channels", "field", "kernel-size"})
    if (!has(required))
      usage(std::string("the option '--") + required + "' is required");
  // Passes (tools/single_conv_layer.cpp:715-735).
  const std::string phase = get("single-phase", "all");
  if (phase != "fwd" && phase != "bwd" && phase != "wu" && phase != "all")
    usage("--single-phase must be fwd, bwd, wu or all");
  const bool inferenceOnly = parseBool(get("inference-only", "false"));
  const bool doFwdPass = phase == "fwd" || phase == "all";
  const bool doBwdPass = !inferenceOnly && (phase == "bwd" || phase == "all");
  bool doWuPass = !inferenceOnly && (phase == "wu" || phase == "all");

  // ---- parameters (tools/single_conv_layer.cpp:768-790) -------------------
  const Shape field = parseShape(get("field"));
  if (field.broadcast)
    usage("--field needs one size per dimension, e.g. {32,32}");
  const size_t n = field.values.size();
  const auto fieldShape = expand<size_t>(field, n, 1);
  const auto kernelShape = expand<size_t>(parseShape(get("kernel-size")), n, 1);
  poplar::Type inputType = parseType(get("data-type", "half"));
  poplar::Type outputType = inputType;
  if (has("input-type"))
    inputType = parseType(get("input-type"));
  if (has("output-type"))
    outputType = parseType(get("output-type"));
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
      inputType, outputType, std::stoul(get("batch-size", "1")), fieldShape,
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
  if (has("fwd-plan-constraints-file")) {
    std::ifstream f(get("fwd-plan-constraints-file"));
    if (!f)
      usage("cannot read '" + get("fwd-plan-constraints-file") + "'");
    std::stringstream ss;
    ss << f.rdbuf();
    options.set("planConstraints", ss.str());
  }
  if (has("fwd-plan-constraints"))
    options.set("planConstraints", get("fwd-plan-constraints"));
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
  if (has("bwd-plan-constraints"))
    bwdOptions.set("planConstraints", get("bwd-plan-constraints"));
  else if (has("fwd-plan-constraints"))
    bwdOptions.set("planConstraints", "");
  poplin::convolutionValidateOptions(bwdOptions);
  // Weight update: the forward options with pass TRAINING_WU
  // (tools/single_conv_layer.cpp:821-824).
  poplar::OptionFlags wuOptions = options;
  wuOptions.set("pass", "TRAINING_WU");
  if (has("wu-plan-constraints"))
    wuOptions.set("planConstraints", get("wu-plan-constraints"));
  else if (has("fwd-plan-constraints"))
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
  if (has("plan-only"))
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
      x = std::ldexp(x, inMeta.scale);
  }
  const auto actBytes = encode(acts, inputType, inMeta);
  const auto weightBytes = encode(weights, inputType, wMeta);
  const auto biasBytes = encode(biases, outputType, {});
  const auto zDeltaBytes = encode(zDeltas, inputType, inMeta);

  // ---- device run ----------------------------------------------------------
  poplin::Stream prog;
  auto in = poplin::createInput(params, options, &cache);
  auto w = poplin::createWeights(params, options, &cache);
  in.metadata = inMeta;
  w.metadata = wMeta;
  std::vector<uint8_t> result(outElems * outputType.size());
  std::vector<uint8_t> first;
  const bool ignoreData = has("ignore-data");
  const unsigned runs = doFwdPass ? 1 + determinismChecks : 0;
  for (unsigned run = 0; run != runs; ++run) {
    if (!ignoreData) {
      poplin::writeTensor(in, actBytes.data(), prog, params, options, &cache);
      poplin::writeTensor(w, weightBytes.data(), prog, params, options, &cache);
    }
    auto out = poplin::convolution(in, w, params, false, prog, options, &cache);
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
    deltas.metadata = inMeta;
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
      poplin::writeTensor(in, actBytes.data(), prog, params, options, &cache);
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
  if (ignoreData) {
    std::cout << "Results not checked (--ignore-data)\n";
    return 0;
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
  return 0;
} catch (const poplar::graph_memory_allocation_error &e) {
  std::cerr << e.what() << std::endl;
  return 77;
} catch (const std::exception &e) {
  std::cerr << "error: " << e.what() << std::endl;
  return 1;
}
