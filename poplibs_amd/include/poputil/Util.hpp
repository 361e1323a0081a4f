// Row-major index helpers (include/poputil/Util.hpp:81-105).
#ifndef poplibs_amd_poputil_Util_hpp
#define poplibs_amd_poputil_Util_hpp
#include <cstddef>
#include <vector>

namespace poputil {

template <class T>
std::vector<T> unflattenIndex(const std::vector<T> &shape, std::size_t index) {
  std::vector<T> coord(shape.size());
  for (std::size_t d = shape.size(); d-- != 0;) {
    coord[d] = static_cast<T>(index % shape[d]);
    index /= shape[d];
  }
  return coord;
}

template <class T>
std::size_t flattenIndex(const std::vector<T> &shape,
                         const std::vector<T> &indices) {
  std::size_t index = 0;
  for (std::size_t d = 0; d != shape.size(); ++d)
    index = index * shape[d] + indices[d];
  return index;
}

} // namespace poputil
#endif
