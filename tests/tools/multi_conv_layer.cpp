// multi_conv_layer - command-line harness for poplin::multiconv: several
// convolutions, each given as ConvParams JSON, run together.
//
// Test infrastructure: it runs them through the C++ layer of this build
// (poplin/MultiConvolution.hpp, hence mxconv_multi_fwd and the gfx950
// kernels) and compares every output with the CPU oracle, as PopLibs'
// tools/multi_conv_layer.cpp compares a device run with
// poplibs_test::conv::convolution / convolutionBackward.  That tool's options
// carry their names here (tools/multi_conv_layer.cpp:74-93): --conv JSON
// (repeatable), --bwd, --enable-convolution-reuse, --report-plan,
// --ignore-data; --tiles-per-ipu, --device-type, --profile are accepted and
// ignored.  --multiconv-options JSON is this build's addition (planType ...).
// The data are random +-1 and the comparison is exact (:197-215, 398-401).
//   exit 0 = match, 1 = mismatch or bad usage, 77 = out of device memory.
#include "poplar/OptionFlags.hpp"
#include "poplar/exceptions.hpp"
#include "poplin/ConvParams.hpp"
#include "poplin/ConvUtil.hpp"
#include "poplin/MultiConvolution.hpp"
#include "poputil/exceptions.hpp"

#include "../../poplibs_amd/src/Json.hpp"
#include "harness_util.hpp"

#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <random>
#include <sstream>

extern "C" {
int oracle_convolution(
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
    unsigned out_chans_per_group, const double *in, const double *kernel,
    const double *biases, double *out, size_t out_elems, int threads);
int oracle_convolution_backward(
    unsigned num_field_dims, const unsigned *fwd_input_field_size,
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
    unsigned out_chans_per_group, const double *deltas_in, const double *kernel,
    double *deltas_out, size_t deltas_out_elems, int threads);
}

namespace {

using poplin::ConvParams;
using poplin::DeviceTensor;

[[noreturn]] void usage(const std::string &message) {
  std::cerr << "error: " << message << "\n"
            << "usage: multi_conv_layer --conv JSON [--conv JSON ...] "
               "[--bwd 0|1] [options]\n"
               "  see the header of tests/tools/multi_conv_layer.cpp for the "
               "option list\n";
  std::exit(1);
}

/// The fp8 metadata a --conv entry may carry next to the parameters
/// (tools/multi_conv_layer.cpp:36-60): formats "F143" / "F152" and scales for
/// the forward input, the weights and the backward input.
struct ConvMetadata {
  poplin::QuarterMetadata fwd, weights, bwd;
};

ConvMetadata parseMetadata(const std::string &text) {
  ConvMetadata m;
  const auto doc = poplibs_amd::json::parse(text);
  auto read = [&](const char *format, const char *scale,
                  poplin::QuarterMetadata &md) {
    for (const auto &member : doc.members) {
      if (member.first == format) {
        if (member.second.text != "F143" && member.second.text != "F152")
          usage(std::string(format) + " must be F143 or F152");
        md.format = member.second.text == "F143"
                        ? poplin::QuarterMetadata::Format::F143
                        : poplin::QuarterMetadata::Format::F152;
      } else if (member.first == scale) {
        md.scale = std::stoi(member.second.text);
      }
    }
  };
  read("fp8FormatFwd", "fp8ScaleFwd", m.fwd);
  read("fp8FormatWeights", "fp8ScaleWeights", m.weights);
  read("fp8FormatBwd", "fp8ScaleBwd", m.bwd);
  return m;
}

std::vector<unsigned> padded(const std::vector<unsigned> &v) {
  auto r = v;
  r.push_back(0); // storage to point at for rank-0 fields
  return r;
}
std::vector<unsigned> padded(const std::vector<std::size_t> &v) {
  std::vector<unsigned> r(v.begin(), v.end());
  r.push_back(0);
  return r;
}
std::vector<unsigned char> padded(const std::vector<bool> &v) {
  std::vector<unsigned char> r(v.begin(), v.end());
  r.push_back(0);
  return r;
}

std::size_t product(const std::vector<std::size_t> &v) {
  std::size_t n = 1;
  for (auto x : v)
    n *= x;
  return n;
}

std::vector<std::size_t> weightsShape(const ConvParams &p) {
  std::vector<std::size_t> s{p.numConvGroups, p.outputChannelsPerConvGroup,
                             p.inputChannelsPerConvGroup};
  s.insert(s.end(), p.kernelShape.begin(), p.kernelShape.end());
  return s;
}

} // namespace

int main(int argc, char **argv) try {
  // --conv repeats, so it is collected before the shared parser (which keeps
  // one value per key) sees the rest.
  std::vector<std::string> convs;
  std::vector<char *> rest{argv[0]};
  for (int i = 1; i < argc; ++i) {
    const std::string arg = argv[i];
    if (arg == "--conv") {
      if (i + 1 >= argc)
        usage("--conv needs a value");
      convs.push_back(argv[++i]);
    } else if (arg.rfind("--conv=", 0) == 0) {
      convs.push_back(arg.substr(7));
    } else {
      rest.push_back(argv[i]);
    }
  }
  auto opt = parseCommandLine(int(rest.size()), rest.data());
  static const char *known[] = {"help", "compile-only", "device-type",
                                "profile", "ignore-data", "tiles-per-ipu",
                                "bwd", "enable-convolution-reuse",
                                "report-plan", "multiconv-options", "seed"};
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
  const bool bwdPass = parseBool(get("bwd", "false"));
  const bool reuse = parseBool(get("enable-convolution-reuse", "true"));
  const bool ignoreData = has("ignore-data");
  std::cout << "got " << convs.size() << " convs" << std::endl;

  poplar::OptionFlags multiConvOptions;
  if (has("multiconv-options")) {
    const auto doc = poplibs_amd::json::parse(get("multiconv-options"));
    if (!doc.isObject())
      usage("--multiconv-options must be a JSON object");
    for (const auto &m : doc.members)
      multiConvOptions.set(m.first, m.second.text);
  }
  poplin::multiconv::validateOptions(multiConvOptions);

  std::vector<ConvParams> fwdParams, bwdParams;
  std::vector<ConvMetadata> metadata;
  for (const auto &conv : convs) {
    std::stringstream ss(conv);
    ConvParams p;
    ss >> p;
    p.validate();
    bwdParams.push_back(poplin::getGradientParams(p));
    fwdParams.push_back(p);
    metadata.push_back(parseMetadata(conv));
  }
  const auto &params = bwdPass ? bwdParams : fwdParams;
  const std::size_t n = params.size();
  poplin::PlanningCache cache;
  const std::vector<poplar::OptionFlags> options(n);
  if (parseBool(get("report-plan", "false")))
    for (std::size_t i = 0; i != n; ++i) {
      std::cout << "Plan:\n";
      poplin::reportPlanInfo(std::cout, params[i], options[i], &cache);
    }
  if (has("compile-only"))
    return 0;

  // ---- operands (tools/multi_conv_layer.cpp:189-232) -----------------------
  poplin::Stream prog;
  std::mt19937 rng(unsigned(std::stoul(get("seed", "5489"))));
  std::bernoulli_distribution coin;
  std::vector<std::vector<double>> hostIn(n), hostW(n);
  std::vector<poplin::multiconv::CreateTensorArgs> createArgs;
  for (std::size_t i = 0; i != n; ++i)
    createArgs.push_back({params[i], options[i], "conv_" + std::to_string(i)});
  std::vector<poplin::multiconv::ConvolutionArgs> convArgs;
  std::vector<DeviceTensor> fwdWeights;
  for (std::size_t i = 0; i != n; ++i) {
    const ConvParams &p = params[i];
    const auto &inMeta = bwdPass ? metadata[i].bwd : metadata[i].fwd;
    hostIn[i].resize(p.batchSize * p.getNumInputChans() *
                     product(p.inputFieldShape));
    // the weights are generated as the forward pass holds them
    hostW[i].resize(product(weightsShape(fwdParams[i])));
    for (auto &x : hostIn[i])
      x = coin(rng) ? 1.0 : -1.0;
    for (auto &x : hostW[i])
      x = coin(rng) ? 1.0 : -1.0;
    const auto inBytes = encode(hostIn[i], p.inputType, inMeta);
    const auto wBytes = encode(hostW[i], p.inputType, metadata[i].weights);
    DeviceTensor input = poplin::multiconv::createInput(
        createArgs, unsigned(i), multiConvOptions, &cache);
    input.metadata = inMeta;
    if (!ignoreData)
      poplin::writeTensor(input, inBytes.data(), prog, p, options[i], &cache);
    DeviceTensor weights;
    if (!bwdPass) {
      weights = poplin::multiconv::createWeights(createArgs, unsigned(i),
                                                 multiConvOptions, &cache);
      weights.metadata = metadata[i].weights;
      if (!ignoreData)
        poplin::writeTensor(weights, wBytes.data(), prog, p, options[i],
                            &cache);
    } else {
      // the forward weights in the external layout; flipped either by
      // multiconv::weightsTransposeChansFlipXY (reuse) or inside the
      // convolution (transposeAndFlipWeights)
      DeviceTensor fwd(p.inputType, weightsShape(fwdParams[i]),
                       DeviceTensor::Layout::External,
                       std::max<std::size_t>(wBytes.size(), 1));
      fwd.metadata = metadata[i].weights;
      if (!ignoreData)
        poplin::writeTensor(fwd, wBytes.data(), prog);
      fwdWeights.push_back(fwd);
      weights = fwd;
      if (reuse) {
        weights = DeviceTensor(p.inputType, weightsShape(p),
                               DeviceTensor::Layout::External,
                               std::max<std::size_t>(wBytes.size(), 1));
        weights.metadata = metadata[i].weights;
      }
    }
    convArgs.push_back({input, weights, p, options[i]});
  }
  std::vector<DeviceTensor> outs;
  if (bwdPass && reuse) {
    poplin::multiconv::weightsTransposeChansFlipXY(
        convArgs, fwdWeights, prog, multiConvOptions, &cache);
    outs = poplin::multiconv::convolution(convArgs, false, prog,
                                          multiConvOptions, &cache);
  } else {
    outs = poplin::multiconv::convolution(convArgs, bwdPass, prog,
                                          multiConvOptions, &cache);
  }
  prog.synchronize();
  if (ignoreData) {
    std::cout << "Results not checked (--ignore-data)\n";
    return 0;
  }

  // ---- host model, exact comparison (:233-285, 383-403) -------------------
  bool matchesModel = true;
  for (std::size_t i = 0; i != n; ++i) {
    const ConvParams &p = params[i], &f = fwdParams[i];
    const std::size_t outElems =
        p.batchSize * p.getNumOutputChans() * product(p.getOutputFieldShape());
    std::vector<double> expected(outElems + 1),
        biases(p.getNumOutputChans() + 1, 0.0);
    hostIn[i].push_back(0);
    hostW[i].push_back(0);
    const auto fs = padded(f.inputFieldShape), ks = padded(f.kernelShape);
    const auto &it = f.inputTransform, &kt = f.kernelTransform;
    const auto &ot = f.outputTransform;
    const auto itl = padded(it.truncationLower), itu = padded(it.truncationUpper),
               idl = padded(it.dilation), ipl = padded(it.paddingLower),
               ipu = padded(it.paddingUpper);
    const auto ktl = padded(kt.truncationLower), ktu = padded(kt.truncationUpper),
               kdl = padded(kt.dilation), kpl = padded(kt.paddingLower),
               kpu = padded(kt.paddingUpper);
    const auto otl = padded(ot.truncationLower), otu = padded(ot.truncationUpper),
               ost = padded(ot.stride), opl = padded(ot.paddingLower),
               opu = padded(ot.paddingUpper);
    const auto fi = padded(it.flip), fk = padded(kt.flip);
    const unsigned nd = unsigned(f.getNumFieldDims());
    int rc;
    if (!bwdPass)
      rc = oracle_convolution(
          nd, fs.data(), itl.data(), itu.data(), idl.data(), ipl.data(),
          ipu.data(), fi.data(), ks.data(), ktl.data(), ktu.data(), kdl.data(),
          kpl.data(), kpu.data(), fk.data(), otl.data(), otu.data(), ost.data(),
          opl.data(), opu.data(), unsigned(f.batchSize),
          unsigned(f.numConvGroups), unsigned(f.inputChannelsPerConvGroup),
          unsigned(f.outputChannelsPerConvGroup), hostIn[i].data(),
          hostW[i].data(), biases.data(), expected.data(), outElems, 8);
    else
      rc = oracle_convolution_backward(
          nd, fs.data(), itl.data(), itu.data(), idl.data(), ipl.data(),
          ipu.data(), fi.data(), ks.data(), ktl.data(), ktu.data(), kdl.data(),
          kpl.data(), kpu.data(), fk.data(), otl.data(), otu.data(), ost.data(),
          opl.data(), opu.data(), unsigned(f.batchSize),
          unsigned(f.numConvGroups), unsigned(f.inputChannelsPerConvGroup),
          unsigned(f.outputChannelsPerConvGroup), hostIn[i].data(),
          hostW[i].data(), expected.data(), outElems, 8);
    if (rc != 0) {
      std::cerr << "host model failed with code " << rc << "\n";
      return 1;
    }
    std::vector<uint8_t> bytes(outElems * p.outputType.size());
    poplin::readTensor(outs[i], bytes.data(), prog, p, options[i], &cache);
    const auto actual = decode(bytes, p.outputType);
    unsigned mismatches = 0;
    for (std::size_t e = 0; e != outElems; ++e)
      if (actual[e] != expected[e] && mismatches++ < 20)
        std::cerr << "mismatch on element conv_" << i << "[" << e
                  << "]: expected=" << expected[e] << " actual=" << actual[e]
                  << "\n";
    matchesModel = matchesModel && mismatches == 0;
  }
  if (!matchesModel) {
    std::cerr << "Validation failed\n";
    return 1;
  }
  std::cout << "Validation passed\n";
  return 0;
} catch (const poplar::graph_memory_allocation_error &e) {
  std::cerr << e.what() << std::endl;
  return 77;
} catch (const std::exception &e) {
  std::cerr << "error: " << e.what() << std::endl;
  return 1;
}
