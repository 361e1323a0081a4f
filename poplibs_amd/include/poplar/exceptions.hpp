// Stand-ins for the two Poplar SDK exceptions the convolution path and its
// harness distinguish (tests/poplin/ConvTest.cpp:684-698,
// tools/single_conv_layer.cpp:1531-1537).
#ifndef poplibs_amd_poplar_exceptions_hpp
#define poplibs_amd_poplar_exceptions_hpp
#include <stdexcept>
#include <string>

namespace poplar {

struct poplar_error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

/// An option key or value that is not recognised.
struct invalid_option : poplar_error {
  using poplar_error::poplar_error;
};

/// Device memory could not be allocated.
struct graph_memory_allocation_error : poplar_error {
  using poplar_error::poplar_error;
};

} // namespace poplar
#endif
