// Pieces the command-line harnesses share: option parsing, conversion of
// host values to and from the device element types, the comparison rule.
// Test infrastructure; each harness defines usage().
#ifndef tests_tools_harness_util_hpp
#define tests_tools_harness_util_hpp
#include "poplar/Type.hpp"
#include "poplin/Convolution.hpp"

#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <string>
#include <vector>

extern "C" {
double oracle_fp8_decode(unsigned code, int format);
unsigned oracle_fp8_encode(double x, int format);
}

namespace {

[[noreturn]] void usage(const std::string &message);

/// "--key value", "--key=value" and bare "--flag" (= "true").
std::map<std::string, std::string> parseCommandLine(int argc, char **argv) {
  std::map<std::string, std::string> opt;
  for (int i = 1; i < argc; ++i) {
    std::string arg = argv[i];
    if (arg.rfind("--", 0) != 0)
      usage("unexpected argument '" + arg + "'");
    arg = arg.substr(2);
    std::string value = "true";
    const auto eq = arg.find('=');
    if (eq != std::string::npos) {
      value = arg.substr(eq + 1);
      arg = arg.substr(0, eq);
    } else if (i + 1 < argc && std::string(argv[i + 1]).rfind("--", 0) != 0) {
      value = argv[++i];
    }
    opt[arg] = value;
  }
  return opt;
}

inline poplar::Type parseType(const std::string &name) {
  if (name == "half")
    return poplar::HALF;
  if (name == "float")
    return poplar::FLOAT;
  if (name == "quarter")
    return poplar::QUARTER;
  usage("unknown type '" + name + "'");
}

inline bool parseBool(const std::string &v) {
  return v == "1" || v == "true" || v == "TRUE" || v == "True";
}

// IEEE binary16 <-> double, round to nearest even.
uint16_t toHalfBits(double d) {
  float f = float(d);
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const int32_t exp = int32_t((x >> 23) & 0xff) - 127 + 15;
  uint32_t mant = x & 0x7fffffu;
  if (((x >> 23) & 0xff) == 0xff)
    return uint16_t(sign | 0x7c00u | (mant ? 0x200u : 0));
  if (exp >= 31)
    return uint16_t(sign | 0x7c00u);
  if (exp <= 0) {
    if (exp < -10)
      return uint16_t(sign);
    mant |= 0x800000u;
    const int shift = 14 - exp;
    uint32_t h = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (h & 1)))
      ++h;
    return uint16_t(sign | h);
  }
  uint32_t h = (uint32_t(exp) << 10) | (mant >> 13);
  const uint32_t rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1)))
    ++h;
  return uint16_t(sign | h);
}

double fromHalfBits(uint16_t h) {
  const int sign = h >> 15, exp = (h >> 10) & 31, mant = h & 1023;
  double v;
  if (exp == 0)
    v = std::ldexp(double(mant), -24);
  else if (exp == 31)
    v = mant ? NAN : INFINITY;
  else
    v = std::ldexp(double(1024 + mant), exp - 25);
  return sign ? -v : v;
}

/// Rounds `values` to `type` in place and returns the device bytes.
inline std::vector<uint8_t> encode(std::vector<double> &values, poplar::Type type,
                            const poplin::QuarterMetadata &md) {
  std::vector<uint8_t> bytes(values.size() * type.size());
  for (size_t i = 0; i != values.size(); ++i) {
    if (type == poplar::FLOAT) {
      const float f = float(values[i]);
      std::memcpy(&bytes[4 * i], &f, 4);
      values[i] = f;
    } else if (type == poplar::HALF) {
      const uint16_t h = toHalfBits(values[i]);
      std::memcpy(&bytes[2 * i], &h, 2);
      values[i] = fromHalfBits(h);
    } else {
      const int fmt = int(md.format);
      const unsigned c =
          oracle_fp8_encode(std::ldexp(values[i], -md.scale), fmt);
      bytes[i] = uint8_t(c);
      values[i] = std::ldexp(oracle_fp8_decode(c, fmt), md.scale);
    }
  }
  return bytes;
}

inline std::vector<double> decode(const std::vector<uint8_t> &bytes,
                           poplar::Type type) {
  std::vector<double> values(bytes.size() / type.size());
  for (size_t i = 0; i != values.size(); ++i) {
    if (type == poplar::FLOAT) {
      float f;
      std::memcpy(&f, &bytes[4 * i], 4);
      values[i] = f;
    } else {
      uint16_t h;
      std::memcpy(&h, &bytes[2 * i], 2);
      values[i] = fromHalfBits(h);
    }
  }
  return values;
}

inline size_t maxContiguousInteger(poplar::Type t) {
  if (t == poplar::HALF)
    return 2048;
  if (t == poplar::FLOAT)
    return 16777216;
  return 16; // quarter
}

/// lib/poplibs_test/Util.cpp:198-217 with boost's strong closeness test.
inline bool isClose(double a, double b, double relTol) {
  if (a == b)
    return true;
  if (std::isnan(a) && std::isnan(b))
    return true;
  if (std::fabs(a) < relTol && std::fabs(b) < relTol)
    return true;
  const double diff = std::fabs(a - b);
  return diff <= relTol * std::fabs(a) && diff <= relTol * std::fabs(b);
}

} // namespace
#endif
