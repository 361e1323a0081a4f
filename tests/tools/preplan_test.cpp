// poplin::preplan and reportPlanEstimatedCosts on the host (no GPU is
// touched): the checks the reference makes of its own preplan
// (tests/poplin/TriangularSolveTest.cpp:82-108: every planned entry is in
// the cache afterwards) and of the plan cost report
// (include/poplin/Convolution.hpp:590-611).  Exit code 0 = all passed.
#include "poplin/ConvPreplan.hpp"
#include "poplin/ConvUtil.hpp"
#include "poplar/exceptions.hpp"
#include "poputil/exceptions.hpp"

#include <iostream>
#include <sstream>
#include <string>

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

int main() {
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
    // three input channels are copied into whole vectors first
    const ConvParams stem = conv(poplar::HALF, 8, 56, 3, 3, 64);
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

  if (failures == 0)
    std::cout << "preplan_test: all checks passed\n";
  return failures == 0 ? 0 : 1;
}
