// poplin::preplan and reportPlanEstimatedCosts on the host (no GPU is
// touched): the checks the reference makes of its own preplan
// (tests/poplin/TriangularSolveTest.cpp:82-108: every planned entry is in
// the cache afterwards) and of the plan cost report
// (include/poplin/Convolution.hpp:590-611).  Exit code 0 = all passed.
#include "poplin/ConvPreplan.hpp"
#include "poplin/ConvUtil.hpp"
#include "poplin/MultiConvolution.hpp"
#include "poplar/exceptions.hpp"
#include "poputil/exceptions.hpp"

#include <cstring>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

using poplin::ConvParams;

static int failures = 0;
#define CHECK(cond)                                                           \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::cerr << __FILE__ << ":" << __LINE__ << ": " #cond "\n";            \
      ++failures;                                                             \
    }                                                                         \
  } while (0)

static ConvParams conv(poplar::Type in, std::size_t batch, std::size_t field,
                       std::size_t kernel, std::size_t ci, std::size_t co,
                       std::size_t groups = 1, unsigned stride = 1) {
  ConvParams p(in, poplar::HALF, batch, {field, field}, {kernel, kernel}, ci,
               co, groups);
  const unsigned pad = unsigned(kernel / 2);
  p.inputTransform.paddingLower = {pad, pad};
  p.inputTransform.paddingUpper = {pad, pad};
  p.outputTransform.stride = {stride, stride};
  return p;
}

static std::string planText(const ConvParams &p,
                            const poplar::OptionFlags &o,
                            poplin::PlanningCache *cache) {
  std::ostringstream os;
  poplin::reportPlanInfo(os, p, o, cache);
  return os.str();
}

// fullyConnectedWeightTranspose on the device against the same exchange of
// axes done on the host: kernels of one tap (a fully connected layer) and of
// three (nothing may be flipped), several groups, half and float.
static int transposeOnDevice() {
  poplin::Stream prog;
  for (const auto type : {poplar::HALF, poplar::FLOAT})
    for (const std::size_t k : {std::size_t(1), std::size_t(3)}) {
      const std::size_t g = 2, ci = 48, co = 80; // of the backward pass
      ConvParams bwd(type, type, 4, {8}, {k}, ci, co, g);
      const std::size_t n = g * ci * co * k;
      const std::size_t es = type == poplar::HALF ? 2 : 4;
      // forward weights [g][ci][co][k]: element (a, i, o, t) holds a small
      // integer both types represent exactly
      std::vector<float> fwdW(n);
      for (std::size_t i = 0; i != n; ++i)
        fwdW[i] = float(int(i * 7919 % 31) - 15);
      std::vector<unsigned char> raw(n * es);
      for (std::size_t i = 0; i != n; ++i) {
        if (type == poplar::FLOAT) {
          std::memcpy(&raw[i * 4], &fwdW[i], 4);
        } else { // integers below 2048 are exact halves
          const float v = fwdW[i];
          unsigned u;
          std::memcpy(&u, &v, 4);
          const unsigned sign = (u >> 16) & 0x8000u;
          const int e = int((u >> 23) & 0xff) - 127 + 15;
          const unsigned short h =
              v == 0.0f ? 0
                        : (unsigned short)(sign | unsigned(e << 10) |
                                           ((u >> 13) & 0x3ffu));
          std::memcpy(&raw[i * 2], &h, 2);
        }
      }
      poplin::DeviceTensor w(type, {g, ci, co, k},
                             poplin::DeviceTensor::Layout::External, n * es);
      poplin::writeTensor(w, raw.data(), prog);
      const poplin::DeviceTensor t =
          poplin::fullyConnectedWeightTranspose(w, bwd, prog);
      CHECK(t.layout() == poplin::DeviceTensor::Layout::PackedWeights);
      CHECK((t.shape() == std::vector<std::size_t>{g, co, ci, k}));
      // The same exchange of axes on the host, given to convolution() in the
      // external layout, must give the bit-identical output: both runs pack
      // for the same plan, so any misplaced element shows.
      std::vector<unsigned char> swappedRaw(n * es);
      for (std::size_t a = 0; a != g; ++a)
        for (std::size_t o = 0; o != co; ++o)
          for (std::size_t i = 0; i != ci; ++i)
            for (std::size_t tap = 0; tap != k; ++tap)
              std::memcpy(
                  &swappedRaw[(((a * co + o) * ci + i) * k + tap) * es],
                  &raw[(((a * ci + i) * co + o) * k + tap) * es], es);
      poplin::DeviceTensor expected(type, {g, co, ci, k},
                                    poplin::DeviceTensor::Layout::External,
                                    n * es);
      poplin::writeTensor(expected, swappedRaw.data(), prog);
      // input: every element a small integer (+-1, +-2 pattern)
      poplin::DeviceTensor in = poplin::createInput(bwd);
      const std::size_t inElems = in.numElements();
      std::vector<unsigned char> inRaw(inElems * es);
      for (std::size_t i = 0; i != inElems; ++i) {
        const float v = float(int(i * 31 % 5) - 2);
        if (type == poplar::FLOAT) {
          std::memcpy(&inRaw[i * 4], &v, 4);
        } else {
          const unsigned short table[5] = {0xc000, 0xbc00, 0x0000, 0x3c00,
                                           0x4000}; // -2 -1 0 1 2
          std::memcpy(&inRaw[i * 2], &table[i * 31 % 5], 2);
        }
      }
      poplin::writeTensor(in, inRaw.data(), prog, bwd);
      const poplin::DeviceTensor viaArranged =
          poplin::convolution(in, t, bwd, false, prog);
      const poplin::DeviceTensor viaHost =
          poplin::convolution(in, expected, bwd, false, prog);
      const std::size_t outBytes = viaHost.numElements() * es;
      std::vector<unsigned char> got(outBytes), want(outBytes);
      poplin::readTensor(viaArranged, got.data(), prog, bwd);
      poplin::readTensor(viaHost, want.data(), prog, bwd);
      prog.synchronize();
      CHECK(std::memcmp(got.data(), want.data(), outBytes) == 0);
      // ... and is not all zeros
      bool any = false;
      for (unsigned char b : want)
        any |= b != 0;
      CHECK(any);
    }
  if (failures == 0)
    std::cout << "preplan_test: device checks passed\n";
  return failures == 0 ? 0 : 1;
}

int main(int argc, char **argv) {
  if (argc > 1 && std::string(argv[1]) == "--device") {
    try {
      return transposeOnDevice();
    } catch (const std::exception &e) {
      std::cerr << "preplan_test --device: " << e.what() << "\n";
      return 1;
    }
  }
  const poplar::OptionFlags fwd{{"pass", "TRAINING_FWD"}};
  const poplar::OptionFlags wu{{"pass", "TRAINING_WU"}};
  const poplar::OptionFlags none;
  const poplar::OptionFlags mmOpts{{"fullyConnectedPass", "INFERENCE_FWD"}};
  const ConvParams c2 = conv(poplar::HALF, 32, 28, 3, 128, 128);
  const ConvParams c3 = conv(poplar::HALF, 32, 56, 1, 64, 256);
  const ConvParams c4 = conv(poplar::HALF, 32, 112, 3, 1, 1, 96, 2);
  // the same convolution with padding no output sees: one canonical form
  ConvParams c2Again = c2;
  const poplar::Target &target = poplar::Target::gfx950();

  std::set<poplin::ConvPlanParams> convs;
  convs.emplace(&target, c2, &fwd);
  convs.emplace(&target, c2, &none); // other options: another plan
  convs.emplace(&target, c3, &fwd);
  convs.emplace(nullptr, c4, &fwd);
  convs.emplace(&target, poplin::getWeightUpdateParams(c2), &wu);
  convs.emplace(nullptr, c2Again, &fwd); // duplicate key through another tuple
  std::set<poplin::MatMulPlanParams> matmuls;
  matmuls.emplace(&target,
                  poplin::MatMulParams{poplar::HALF, poplar::HALF,
                                       {1, 512, 1024}, {1, 1024, 768}},
                  &mmOpts);
  matmuls.emplace(nullptr,
                  poplin::MatMulParams{poplar::HALF, poplar::FLOAT,
                                       {4, 64, 256}, {4, 256, 128}},
                  &mmOpts);

  poplin::PlanningCache cache;
  poplin::preplan({}, {}, cache);
  CHECK(cache.size() == 0);
  poplin::preplan(convs, matmuls, cache);
  CHECK(cache.size() == 7); // 5 distinct convolutions + 2 multiplications
  poplin::preplan(convs, matmuls, cache); // all there already
  CHECK(cache.size() == 7);

  // what is used afterwards finds its plan in the cache, and it is the plan
  // that planning it alone makes
  for (const auto &entry : convs) {
    const std::string viaCache =
        planText(std::get<1>(entry), *std::get<2>(entry), &cache);
    CHECK(viaCache == planText(std::get<1>(entry), *std::get<2>(entry),
                               nullptr));
  }
  {
    std::ostringstream os;
    poplin::matMulReportPlan(os, poplar::HALF, poplar::HALF, {512, 1024},
                             {1024, 768}, mmOpts, &cache);
    poplin::matMulGroupedReportPlan(os, poplar::HALF, poplar::FLOAT,
                                    {4, 64, 256}, {4, 256, 128}, mmOpts,
                                    &cache);
  }
  CHECK(cache.size() == 7);

  // matMulGetConvPlanParams: one set of convolution options per options
  // pointer, the multiplication as the convolution matMul plans
  {
    poplin::MatMulToConvOptions made;
    const auto asConvs = poplin::matMulGetConvPlanParams(matmuls, made);
    CHECK(asConvs.size() == 2 && made.size() == 1);
    for (const auto &entry : asConvs) {
      const ConvParams &p = std::get<1>(entry);
      CHECK(p.getNumFieldDims() == 1 && p.kernelShape[0] == 1);
      CHECK(std::get<2>(entry) == &made.begin()->second);
    }
  }

  // an invalid entry: the error planning it alone gives, and a cache that
  // holds none of the call's plans
  {
    poplin::PlanningCache fresh;
    const poplar::OptionFlags bad{{"partialsType", "double"}};
    std::set<poplin::ConvPlanParams> withBad{
        std::make_tuple(&target, c2, &fwd), std::make_tuple(&target, c3, &bad)};
    bool threw = false;
    try {
      poplin::preplan(withBad, {}, fresh);
    } catch (const poplar::invalid_option &) {
      threw = true;
    } catch (const poputil::poplibs_error &) {
      threw = true;
    }
    CHECK(threw);
    CHECK(fresh.size() == 0);
    ConvParams quarterOut = c2;
    quarterOut.outputType = poplar::QUARTER;
    threw = false;
    try {
      poplin::preplan({std::make_tuple(&target, quarterOut, &fwd)}, {}, fresh);
    } catch (const poputil::poplibs_error &) {
      threw = true;
    }
    CHECK(threw && fresh.size() == 0);
    threw = false;
    try {
      poplin::preplan({std::make_tuple(&target, c2, nullptr)}, {}, fresh);
    } catch (const poputil::poplibs_error &) {
      threw = true;
    }
    CHECK(threw);
  }

  // estimated costs.  Measured on MI355X: c2 8.5 us, c3 11.6 us, c4 17.9 us;
  // the estimate is within a quarter of each, in cycles at 2.1 GHz.
  auto us = [&](const ConvParams &p, const poplar::OptionFlags &o) {
    const poplin::PlanCosts costs =
        poplin::reportPlanEstimatedCosts(p, o, &cache);
    CHECK(costs.cycles != poplin::PlanCosts::unknown);
    return double(costs.cycles) / 2100.0;
  };
  CHECK(us(c2, fwd) > 8.5 * 0.75 && us(c2, fwd) < 8.5 * 1.25);
  CHECK(us(c3, fwd) > 11.6 * 0.75 && us(c3, fwd) < 11.6 * 1.25);
  CHECK(us(c4, fwd) > 17.9 * 0.75 && us(c4, fwd) < 17.9 * 1.25);
  CHECK(cache.size() == 7);
  // more work costs more; no temporary memory for these
  CHECK(us(conv(poplar::HALF, 128, 28, 3, 128, 128), fwd) > 3 * us(c2, fwd));
  CHECK(poplin::reportPlanEstimatedCosts(c2, fwd).memory == 0);
  // a K split sums fp32 partial tiles from the workspace: temporary memory
  {
    const ConvParams deep = conv(poplar::HALF, 8, 28, 3, 128, 128);
    const std::string text = planText(deep, fwd, nullptr);
    const poplin::PlanCosts costs =
        poplin::reportPlanEstimatedCosts(deep, fwd);
    if (text.find("K split into parts") != std::string::npos)
      CHECK(costs.memory > 0);
    CHECK(costs.cycles != poplin::PlanCosts::unknown);
  }
  // the generic kernel is outside the cost model
  {
    const ConvParams odd = conv(poplar::FLOAT, 1, 5, 3, 3, 5);
    const std::string text = planText(odd, none, nullptr);
    const poplin::PlanCosts costs = poplin::reportPlanEstimatedCosts(odd, none);
    if (text.find("generic direct") != std::string::npos)
      CHECK(costs.cycles == poplin::PlanCosts::unknown);
  }

  // the same estimate by phase (include/poplin/Convolution.hpp:613-676)
  {
    using poplin::internal::DetailedPlanCosts;
    auto sumOfPhases = [](const DetailedPlanCosts &d) {
      std::size_t sum = 0;
      d.apply([&](const poplin::PlanCosts &c) { sum += c.cycles; },
              /*includeTotal=*/false);
      return sum;
    };
    // one kernel, nothing else: all of it is compute, 256 workgroups at once
    const DetailedPlanCosts plain =
        poplin::internal::reportDetailedPlanEstimatedCosts(c2, fwd, &cache);
    CHECK(plain.total.cycles ==
          poplin::reportPlanEstimatedCosts(c2, fwd, &cache).cycles);
    CHECK(plain.compute.cycles == plain.total.cycles);
    CHECK(plain.rearrangement.cycles == 0 && plain.reduction.cycles == 0);
    CHECK(sumOfPhases(plain) == plain.total.cycles);
    CHECK(plain.parallelSplit >= 1 && plain.parallelSplit <= 2 * 256);
    CHECK(plain.serialSplit >= 1);
    // a K split: the sum of the partial tiles is the reduction and owns the
    // temporary memory
    const ConvParams deep = conv(poplar::HALF, 8, 28, 3, 128, 128);
    const DetailedPlanCosts split =
        poplin::internal::reportDetailedPlanEstimatedCosts(deep, fwd);
    const poplin::PlanCosts whole = poplin::reportPlanEstimatedCosts(deep, fwd);
    CHECK(split.total.cycles == whole.cycles);
    CHECK(split.total.memory == whole.memory);
    CHECK(sumOfPhases(split) == split.total.cycles);
    if (planText(deep, fwd, nullptr).find("K split into parts") !=
        std::string::npos) {
      CHECK(split.reduction.cycles > 0);
      CHECK(split.reduction.memory == whole.memory);
    }
    // six input channels are copied into whole vectors first
    const ConvParams stem = conv(poplar::HALF, 8, 56, 3, 6, 64);
    const DetailedPlanCosts padded =
        poplin::internal::reportDetailedPlanEstimatedCosts(stem, fwd);
    if (planText(stem, fwd, nullptr).find("generic direct") ==
        std::string::npos) {
      CHECK(padded.rearrangement.cycles > 0);
      CHECK(padded.rearrangement.memory > 0);
      CHECK(padded.rearrangement.memory <= padded.total.memory);
      CHECK(sumOfPhases(padded) == padded.total.cycles);
    }
    // text form: two numbers, then a pair per phase and the total; reads back
    std::stringstream ss;
    ss << split;
    std::size_t lines = 0;
    for (char ch : ss.str())
      lines += ch == '\n';
    CHECK(lines == 14);
    DetailedPlanCosts back;
    ss >> back;
    CHECK(back.parallelSplit == split.parallelSplit);
    CHECK(back.serialSplit == split.serialSplit);
    CHECK(back.compute.cycles == split.compute.cycles);
    CHECK(back.reduction.memory == split.reduction.memory);
    CHECK(back.total.cycles == split.total.cycles);
    // serialSplitOnly visits the eight per-slice phases
    std::size_t visited = 0;
    split.apply([&](const poplin::PlanCosts &) { ++visited; }, false, true);
    CHECK(visited == 8);
    // outside the cost model
    const ConvParams odd = conv(poplar::FLOAT, 1, 5, 3, 3, 5);
    if (planText(odd, none, nullptr).find("generic direct") !=
        std::string::npos) {
      const DetailedPlanCosts d =
          poplin::internal::reportDetailedPlanEstimatedCosts(odd, none);
      CHECK(d.total.cycles == poplin::PlanCosts::unknown);
      CHECK(d.compute.cycles == poplin::PlanCosts::unknown);
    }
  }

  // perfect cycle counts: MACs over what the matrix cores retire per cycle
  // (include/poplin/Convolution.hpp:34-77)
  {
    const double macs = 32.0 * 28 * 28 * 128 * 128 * 9; // c2, padding MACs in
    const double perfect = poplin::getFwdPerfectCycleCount(c2);
    CHECK(perfect == double(poplin::getFwdFlops(c2) / 2) / (512.0 * 4 * 256));
    CHECK(perfect < macs / (512.0 * 4 * 256) && perfect > 6000);
    CHECK(poplin::getBwdPerfectCycleCount(c2) == perfect);
    CHECK(poplin::getWuPerfectCycleCount(c2) == perfect);
    // fp8 retires twice, fp32 a sixteenth of fp16's MACs per cycle
    const ConvParams q = conv(poplar::QUARTER, 32, 28, 3, 128, 128);
    ConvParams f = c2;
    f.inputType = f.outputType = poplar::FLOAT;
    CHECK(poplin::getFwdPerfectCycleCount(q) * 2 == perfect);
    CHECK(poplin::getFwdPerfectCycleCount(f) == perfect * 16);
    // against the estimate: no plan is faster than perfect
    CHECK(double(poplin::reportPlanEstimatedCosts(c2, fwd, &cache).cycles) >
          perfect);
  }

  // preplanConvolutions, the older name: convolutions only, same cache
  {
    poplin::PlanningCache old;
    poplin::preplanConvolutions(convs, old);
    CHECK(old.size() == 5);
    poplin::preplanConvolutions({}, old);
    CHECK(old.size() == 5);
  }

  // ... and preplanMatMuls with the older cache type
  {
    poplin::matmul::PlanningCache old;
    poplin::preplanMatMuls(matmuls, old);
    CHECK(old.size() == 2);
    CHECK(&old.getImpl() == &old);
  }

  // fullyConnectedWeightTranspose refuses what the reference refuses, before
  // anything touches a device
  {
    bool threw = false;
    try {
      poplin::Stream defaultStream(nullptr);
      poplin::fullyConnectedWeightTranspose(poplin::DeviceTensor(), c2,
                                            defaultStream);
    } catch (const poputil::poplibs_error &e) {
      threw = std::string(e.what()).find("expects a 1-d convolution") !=
              std::string::npos;
    }
    CHECK(threw);
    threw = false;
    try {
      poplin::Stream defaultStream(nullptr);
      ConvParams fc(poplar::HALF, poplar::HALF, 4, {1}, {1}, 64, 32, 1);
      poplin::fullyConnectedWeightTranspose(poplin::DeviceTensor(), fc,
                                            defaultStream);
    } catch (const poputil::poplibs_error &e) {
      threw = std::string(e.what()).find("forward pass's weights") !=
              std::string::npos;
    }
    CHECK(threw);
  }

  // a parallel multi-convolution whose entries disagree on
  // insertTransformsCycleCountProgs is refused, a serial one is not asked
  // (tests/poplin/MultiConvolutionTest.cpp:84-130,
  // lib/poplin/MultiConvolution.cpp:155-173); decided before any tensor is
  // looked at
  {
    ConvParams a(poplar::HALF, poplar::HALF, 4, {8, 8}, {4, 4}, 1, 1, 10);
    ConvParams b(poplar::FLOAT, poplar::FLOAT, 4, {5, 5}, {1, 1}, 11, 5, 1);
    const std::vector<poplin::multiconv::ConvolutionArgs> args{
        {poplin::DeviceTensor(), poplin::DeviceTensor(), a,
         {{"insertTransformsCycleCountProgs", "true"}}},
        {poplin::DeviceTensor(), poplin::DeviceTensor(), b,
         {{"insertTransformsCycleCountProgs", "false"}}}};
    poplin::Stream defaultStream(nullptr);
    std::string message;
    try {
      poplin::multiconv::convolution(args, false, defaultStream,
                                     {{"planType", "parallel"}});
    } catch (const poputil::poplibs_error &e) {
      message = e.what();
    }
    CHECK(message.find("<insertTransformsCycleCountProgs>") !=
          std::string::npos);
    message.clear();
    try { // serial: gets as far as the (absent) tensors' shapes
      poplin::multiconv::convolution(args, false, defaultStream,
                                     {{"planType", "serial"}});
    } catch (const poputil::poplibs_error &e) {
      message = e.what();
    }
    CHECK(message.find("does not have the shape") != std::string::npos);
  }

  if (failures == 0)
    std::cout << "preplan_test: all checks passed\n";
  return failures == 0 ? 0 : 1;
}
