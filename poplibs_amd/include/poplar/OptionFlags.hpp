// Minimal stand-in for poplar::OptionFlags: an ordered string -> string map.
#ifndef poplibs_amd_poplar_OptionFlags_hpp
#define poplibs_amd_poplar_OptionFlags_hpp
#include <initializer_list>
#include <map>
#include <string>
#include <utility>

namespace poplar {

class OptionFlags {
  std::map<std::string, std::string> flags_;

public:
  OptionFlags() = default;
  OptionFlags(
      std::initializer_list<std::pair<const std::string, std::string>> init)
      : flags_(init) {}
  void set(const std::string &key, const std::string &value) {
    flags_[key] = value;
  }
  void set(
      std::initializer_list<std::pair<const std::string, std::string>> init) {
    for (const auto &kv : init)
      flags_[kv.first] = kv.second;
  }
  void clear() { flags_.clear(); }
  auto begin() const { return flags_.begin(); }
  auto end() const { return flags_.end(); }
  std::size_t size() const { return flags_.size(); }
  friend bool operator==(const OptionFlags &a, const OptionFlags &b) {
    return a.flags_ == b.flags_;
  }
  friend bool operator<(const OptionFlags &a, const OptionFlags &b) {
    return a.flags_ < b.flags_;
  }
};

} // namespace poplar
#endif
