// Minimal stand-in for the Poplar SDK's element-type handle, limited to the
// three types a poplin convolution accepts (lib/poplin/ConvValidation.cpp:
// 24-32).  The Poplar SDK itself is not part of PopLibs.
#ifndef poplibs_amd_poplar_Type_hpp
#define poplibs_amd_poplar_Type_hpp
#include <cstddef>
#include <iosfwd>
#include <string>

namespace poplar {

class Type {
  int id_;

public:
  constexpr Type() : id_(2) {}
  constexpr explicit Type(int id) : id_(id) {}
  constexpr int id() const { return id_; }
  /// "quarter", "half" or "float": the spellings the ConvParams JSON reader
  /// accepts (lib/poplin/ConvParams.cpp:365-368).
  std::string toString() const;
  /// Bytes per element.
  std::size_t size() const { return id_ == 0 ? 1 : id_ == 1 ? 2 : 4; }
  friend constexpr bool operator==(Type a, Type b) { return a.id_ == b.id_; }
  friend constexpr bool operator!=(Type a, Type b) { return a.id_ != b.id_; }
  friend constexpr bool operator<(Type a, Type b) { return a.id_ < b.id_; }
};

constexpr Type QUARTER{0};
constexpr Type HALF{1};
constexpr Type FLOAT{2};

std::ostream &operator<<(std::ostream &os, const Type &t);

} // namespace poplar
#endif
