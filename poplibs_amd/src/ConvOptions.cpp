#include "ConvOptions.hpp"
#include "poplar/exceptions.hpp"

#include <cstdlib>
#include <set>
#include <sstream>

namespace poplin {

using poplar::invalid_option;
using poplibs_amd::json::Value;

const char *toString(Pass p) {
  static const char *names[] = {
      "NONE",        "NONE_MATMUL",      "INFERENCE_FWD",   "TRAINING_FWD",
      "TRAINING_BWD", "TRAINING_WU",     "FC_INFERENCE_FWD", "FC_TRAINING_FWD",
      "FC_TRAINING_BWD", "FC_TRAINING_WU"};
  return names[int(p)];
}

namespace {

[[noreturn]] void badValue(const std::string &key, const std::string &value,
                           const std::string &expected) {
  throw invalid_option("Invalid value '" + value + "' for option '" + key +
                       "'. " + expected);
}

Pass parsePass(const std::string &key, const std::string &v) {
  for (int i = 0; i <= int(Pass::FC_TRAINING_WU); ++i)
    if (v == toString(Pass(i)))
      return Pass(i);
  badValue(key, v, "Expected a pass name such as INFERENCE_FWD or TRAINING_FWD");
}

poplar::Type parsePartialsType(const std::string &key, const std::string &v) {
  if (v == "half")
    return poplar::HALF;
  if (v == "float")
    return poplar::FLOAT;
  badValue(key, v, "Valid values are 'half' and 'float'");
}

void parseBool(const std::string &key, const std::string &v) {
  if (v != "true" && v != "false")
    badValue(key, v, "Valid values are 'true' and 'false'");
}

double parseDouble(const std::string &key, const std::string &v, double low) {
  char *end = nullptr;
  const double d = std::strtod(v.c_str(), &end);
  if (v.empty() || *end != '\0')
    badValue(key, v, "Expected a number");
  if (d < low)
    badValue(key, v, "Value is below the minimum of " + std::to_string(low));
  return d;
}

// ---- planConstraints (lib/poplin/ConvOptions.cpp:193-329) -----------------

void requireObject(const std::string &path, const Value &v) {
  if (!v.isObject())
    throw invalid_option("'" + path + "': Must be an object");
}
unsigned requireUnsigned(const std::string &path, const Value &v) {
  unsigned long long u;
  if (v.isObject() || v.isArray() || !v.asUnsigned(u))
    throw invalid_option("'" + path + "': Not a valid unsigned integer");
  return unsigned(u);
}
void requireBool(const std::string &path, const Value &v) {
  bool b;
  if (v.isObject() || v.isArray() || !v.asBool(b))
    throw invalid_option("'" + path + "': Not a valid boolean");
}
void requireUnsignedArray(const std::string &path, const Value &v) {
  if (!v.isArray())
    throw invalid_option("'" + path + "': Must be an array");
  for (const Value &item : v.items)
    requireUnsigned(path, item);
}
void requireIndex(const std::string &path, const std::string &index) {
  char *end = nullptr;
  const long long level = std::strtoll(index.c_str(), &end, 10);
  if (index.empty() || end == index.c_str())
    throw invalid_option("'" + path + "': Index not an integer");
  if (level < 0)
    throw invalid_option("'" + path + "': Index is negative");
}

void checkTransform(const std::string &path, const Value &v) {
  requireObject(path, v);
  for (const auto &m : v.members) {
    const std::string sub = path + "." + m.first;
    if (m.first == "swapOperands")
      requireBool(sub, m.second);
    else if (m.first == "expandDims" || m.first == "outChanFlattenDims" ||
             m.first == "combineConvGroupsFactor")
      requireUnsignedArray(sub, m.second);
    else
      throw invalid_option("'" + sub + "': " + m.first +
                           " is not currently handled or does not exist");
  }
}

void checkPartition(const std::string &path, const Value &v) {
  requireObject(path, v);
  for (const auto &m : v.members) {
    const std::string sub = path + "." + m.first;
    if (m.first == "convGroupSplit" || m.first == "batchSplit") {
      requireUnsigned(sub, m.second);
    } else if (m.first == "fieldSplit" || m.first == "kernelSplit") {
      requireObject(sub, m.second);
      for (const auto &dim : m.second.members) {
        requireIndex(sub + "." + dim.first, dim.first);
        requireUnsigned(sub + "." + dim.first, dim.second);
      }
    } else if (m.first == "inChanSplit" || m.first == "outChanSplit") {
      requireObject(sub, m.second);
      for (const auto &s : m.second.members) {
        if (s.first != "parallel" && s.first != "serial")
          throw invalid_option("'" + sub + "." + s.first + "': " + s.first +
                               " is not either 'parallel' or 'serial'");
        requireUnsigned(sub + "." + s.first, s.second);
      }
    } else {
      throw invalid_option("'" + sub + "': " + m.first +
                           " is not currently handled or does not exist");
    }
  }
}

void checkLevel(const std::string &path, const Value &v) {
  requireObject(path, v);
  for (const auto &m : v.members) {
    const std::string sub = path + "." + m.first;
    if (m.first == "transform")
      checkTransform(sub, m.second);
    else if (m.first == "partition")
      checkPartition(sub, m.second);
    else
      throw invalid_option("'" + sub + "': " + m.first +
                           " is not a valid sub-domain of the plan. Must be "
                           "either 'transform' or 'partition'");
  }
}

PlanConstraints::Method checkMethod(const std::string &path, const Value &v) {
  requireObject(path, v);
  auto method = PlanConstraints::Method::ANY;
  for (const auto &m : v.members) {
    if (m.first == "type") {
      if (m.second.kind != Value::String)
        throw invalid_option("'" + path + "': Not a valid string");
      const std::string &t = m.second.text;
      if (t == "AMP")
        method = PlanConstraints::Method::AMP;
      else if (t == "SLIC")
        method = PlanConstraints::Method::SLIC;
      else if (t == "HMAC")
        method = PlanConstraints::Method::HMAC;
      else if (t == "VMAC")
        method = PlanConstraints::Method::VMAC;
      else if (t == "OUTER_PRODUCT")
        method = PlanConstraints::Method::OUTER_PRODUCT;
      else
        throw invalid_option("'" + path + "': Not a valid method type");
    } else if (m.first == "useLimitedVersion") {
      requireBool(m.first, m.second);
    } else if (m.first == "convUnits" || m.first == "convUnitChainsRequired" ||
               m.first == "windowWidth") {
      requireUnsigned(m.first, m.second);
    }
  }
  return method;
}

void checkGfx950(const std::string &path, const Value &v, PlanConstraints &pc) {
  requireObject(path, v);
  for (const auto &m : v.members) {
    const std::string sub = path + "." + m.first;
    if (m.first == "kernel") {
      const std::string &k = m.second.text;
      if (m.second.kind != Value::String ||
          (k != "generic" && k != "igemm" && k != "depthwise"))
        throw invalid_option("'" + sub +
                             "': Must be 'generic', 'igemm' or 'depthwise'");
      pc.kernel = k;
    } else if (m.first == "blockM") {
      pc.blockM = requireUnsigned(sub, m.second);
    } else if (m.first == "blockN") {
      pc.blockN = requireUnsigned(sub, m.second);
    } else if (m.first == "blockK") {
      pc.blockK = requireUnsigned(sub, m.second);
    } else if (m.first == "splitK") {
      pc.splitK = requireUnsigned(sub, m.second);
    } else if (m.first == "stages") {
      pc.stages = requireUnsigned(sub, m.second);
    } else if (m.first == "patch") {
      const unsigned v = requireUnsigned(sub, m.second);
      if (v > 2)
        throw invalid_option("'" + sub + "': Must be 0, 1 or 2");
      pc.patch = int(v);
    } else if (m.first == "rowRing") {
      const unsigned v = requireUnsigned(sub, m.second);
      if (v > 1)
        throw invalid_option("'" + sub + "': Must be 0 or 1");
      pc.rowRing = int(v);
    } else if (m.first == "pointwise") {
      const unsigned v = requireUnsigned(sub, m.second);
      if (v > 1)
        throw invalid_option("'" + sub + "': Must be 0 or 1");
      pc.pointwise = int(v);
    } else if (m.first == "thinInput") {
      const unsigned v = requireUnsigned(sub, m.second);
      if (v > 1)
        throw invalid_option("'" + sub + "': Must be 0 or 1");
      pc.thinInput = int(v);
    } else if (m.first == "weightDeltas") {
      const unsigned v = requireUnsigned(sub, m.second);
      if (v > 2)
        throw invalid_option("'" + sub + "': Must be 0, 1 or 2");
      pc.weightDeltas = int(v);
    } else if (m.first == "chanTiles") {
      pc.chanTiles = requireUnsigned(sub, m.second);
      if (pc.chanTiles < 1 || pc.chanTiles > 4)
        throw invalid_option("'" + sub + "': Must be 1 to 4");
    } else if (m.first == "tileH") {
      pc.tileH = requireUnsigned(sub, m.second);
    } else if (m.first == "tileW") {
      pc.tileW = requireUnsigned(sub, m.second);
    } else {
      throw invalid_option("'" + sub + "': " + m.first +
                           " is not a gfx950 plan constraint");
    }
  }
}

PlanConstraints parsePlanConstraints(const std::string &text) {
  PlanConstraints pc;
  pc.text = text;
  if (text.empty())
    return pc;
  Value root;
  try {
    root = poplibs_amd::json::parse(text);
  } catch (const poplibs_amd::json::ParseError &e) {
    throw invalid_option(std::string("planConstraints: ") + e.what());
  }
  if (!root.isObject())
    throw invalid_option("Plan constraints must be an object");
  for (const auto &m : root.members) {
    if (m.first == "method")
      pc.method = checkMethod(m.first, m.second);
    else if (m.first == "convGroupsPerGroup")
      pc.convGroupsPerGroup = requireUnsigned(m.first, m.second);
    else if (m.first == "inChansPerGroup" || m.first == "partialChansPerGroup")
      requireUnsigned(m.first, m.second);
    else if (m.first == "gfx950")
      checkGfx950(m.first, m.second, pc);
    else {
      requireIndex(m.first, m.first);
      checkLevel(m.first, m.second);
    }
  }
  return pc;
}

} // namespace

ConvOptions::ConvOptions(
    const std::vector<std::pair<std::string, std::string>> &flags) {
  static const std::set<std::string> boolKeys = {
      "use128BitConvUnitLoad",
      "enableMultiStageReduce",
      "enableFastReduce",
      "remapOutputTensor",
      "enableConvDithering",
      "disableTransformations",
      "insertTransformsCycleCountProgs",
      "experimental.convTransformsEstimates",
      "gatherConvOutput",
      "experimental.slicVmac16",
      "disableSRForAMPVertices",
      "enableTileLevelExpandDims"};
  for (const auto &kv : flags) {
    const std::string &key = kv.first, &value = kv.second;
    if (key == "availableMemoryProportion")
      availableMemoryProportion = parseDouble(key, value, 0.);
    else if (key == "pass")
      pass = parsePass(key, value);
    else if (key == "partialsType")
      partialsType = parsePartialsType(key, value);
    else if (key == "partialsType.interTile")
      interTilePartialsType = parsePartialsType(key, value);
    else if (key == "partialsType.interIPU")
      interIpuPartialsType = parsePartialsType(key, value);
    else if (key == "planConstraints")
      planConstraints = parsePlanConstraints(value);
    else if (key == "planConstraintsOutputFilename")
      planConstraintsOutputFilename = value;
    else if (boolKeys.count(key))
      parseBool(key, value); // IPU-only switches: checked, then ignored
    else
      throw invalid_option("Unrecognised option '" + key + "'");
  }
}

std::string ConvOptions::key() const {
  std::ostringstream os;
  os << toString(pass) << '|' << partialsType.toString() << '|'
     << planConstraints.text;
  return os.str();
}

namespace {

bool isFullyConnected(Pass p) {
  return p == Pass::FC_INFERENCE_FWD || p == Pass::FC_TRAINING_FWD ||
         p == Pass::FC_TRAINING_BWD || p == Pass::FC_TRAINING_WU;
}

} // namespace

bool isWeightUpdatePass(Pass p) {
  return p == Pass::TRAINING_WU || p == Pass::FC_TRAINING_WU;
}

std::string getPlanConstraintsOutputFile(const ConvOptions &options) {
  if (options.planConstraintsOutputFilename.empty())
    return {};
  std::string path = options.planConstraintsOutputFilename;
  switch (options.pass) {
  case Pass::INFERENCE_FWD:
  case Pass::TRAINING_FWD:
  case Pass::FC_INFERENCE_FWD:
  case Pass::FC_TRAINING_FWD:
    path += "_FWD";
    break;
  case Pass::TRAINING_BWD:
  case Pass::FC_TRAINING_BWD:
    path += "_BWD";
    break;
  case Pass::TRAINING_WU:
  case Pass::FC_TRAINING_WU:
    path += "_WU";
    break;
  case Pass::NONE:
  case Pass::NONE_MATMUL:
    break;
  }
  return path + ".json";
}

ConvOptions getWeightUpdateOptions(ConvOptions fwdOptions) {
  fwdOptions.pass = isFullyConnected(fwdOptions.pass) ? Pass::FC_TRAINING_WU
                                                      : Pass::TRAINING_WU;
  return fwdOptions;
}

ConvOptions getGradientOptions(ConvOptions fwdOptions) {
  fwdOptions.pass = isFullyConnected(fwdOptions.pass) ? Pass::FC_TRAINING_BWD
                                                      : Pass::TRAINING_BWD;
  return fwdOptions;
}

} // namespace poplin
