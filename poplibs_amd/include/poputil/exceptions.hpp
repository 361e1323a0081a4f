// poputil::poplibs_error, the exception PopLibs raises for invalid shapes and
// parameters (include/poputil/exceptions.hpp:17-21).
#ifndef poplibs_amd_poputil_exceptions_hpp
#define poplibs_amd_poputil_exceptions_hpp
#include <stdexcept>
#include <string>

namespace poputil {

struct poplibs_error : std::runtime_error {
  std::string type = "poplibs_error";
  explicit poplibs_error(const std::string &s) : std::runtime_error(s) {}
  explicit poplibs_error(const char *s) : std::runtime_error(s) {}
};

} // namespace poputil
#endif
