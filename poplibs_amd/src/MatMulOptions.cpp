#include "MatMulOptions.hpp"
#include "poplar/exceptions.hpp"

#include <cstdlib>
#include <map>

namespace poplin {

namespace {

bool parseBool(const std::string &key, const std::string &value) {
  if (value == "true")
    return true;
  if (value == "false")
    return false;
  throw poplar::invalid_option("Invalid value '" + value + "' for option '" +
                               key + "': must be true or false");
}

} // namespace

OptionList matMulToConvOptions(const OptionList &matMulOptions) {
  // Defaults of MatMulOptions (lib/poplin/MatMul.cpp:54-78).
  std::string partialsType = "float", pass = "NONE", planConstraints;
  double availableMemoryProportion = .6;
  std::map<std::string, bool> switches{
      {"inputRHSIsPreArranged", false}, {"use128BitConvUnitLoad", false},
      {"enableMultiStageReduce", true}, {"enableFastReduce", false},
      {"remapOutputTensor", true},      {"gatherOutput", false},
      {"disableSRForAMPVertices", false}};
  for (const auto &kv : matMulOptions) {
    const std::string &key = kv.first, &value = kv.second;
    if (key == "partialsType") {
      if (value != "half" && value != "float")
        throw poplar::invalid_option("Invalid value '" + value +
                                     "' for option 'partialsType': must be "
                                     "half or float");
      partialsType = value;
    } else if (key == "fullyConnectedPass") {
      if (value != "NONE" && value != "INFERENCE_FWD" &&
          value != "TRAINING_FWD" && value != "TRAINING_BWD" &&
          value != "TRAINING_WU")
        throw poplar::invalid_option(
            "Invalid value '" + value +
            "' for option 'fullyConnectedPass': must be NONE, INFERENCE_FWD, "
            "TRAINING_FWD, TRAINING_BWD or TRAINING_WU");
      pass = value;
    } else if (key == "availableMemoryProportion") {
      char *end = nullptr;
      availableMemoryProportion = std::strtod(value.c_str(), &end);
      if (value.empty() || *end != '\0' || availableMemoryProportion < 0.)
        throw poplar::invalid_option(
            "Invalid value '" + value +
            "' for option 'availableMemoryProportion': must be a number >= 0");
    } else if (key == "planConstraints") {
      planConstraints = value;
    } else if (switches.count(key)) {
      switches[key] = parseBool(key, value);
    } else {
      throw poplar::invalid_option("Unrecognised option '" + key + "'");
    }
  }
  auto flag = [&](const char *k) {
    return std::string(switches[k] ? "true" : "false");
  };
  OptionList conv;
  conv.emplace_back("partialsType", partialsType);
  conv.emplace_back("availableMemoryProportion",
                    std::to_string(availableMemoryProportion));
  conv.emplace_back("use128BitConvUnitLoad", flag("use128BitConvUnitLoad"));
  conv.emplace_back("enableMultiStageReduce", flag("enableMultiStageReduce"));
  conv.emplace_back("enableFastReduce", flag("enableFastReduce"));
  conv.emplace_back("remapOutputTensor", flag("remapOutputTensor"));
  conv.emplace_back("gatherConvOutput", flag("gatherOutput"));
  conv.emplace_back("disableSRForAMPVertices", flag("disableSRForAMPVertices"));
  conv.emplace_back("planConstraints", planConstraints);
  conv.emplace_back("pass", pass == "NONE" ? "NONE_MATMUL" : "FC_" + pass);
  return conv;
}

} // namespace poplin
