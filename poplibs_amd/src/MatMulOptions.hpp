// Matrix-multiplication options (lib/poplin/MatMul.cpp:40-157) and their
// translation into convolution options (getConvOptionFlags, :159-195).
#ifndef poplibs_amd_MatMulOptions_hpp
#define poplibs_amd_MatMulOptions_hpp
#include <string>
#include <utility>
#include <vector>

namespace poplin {

using OptionList = std::vector<std::pair<std::string, std::string>>;

/// Checks every key and value of a matMul option set (throws
/// poplar::invalid_option) and returns the convolution options the
/// multiplication is planned with: partialsType, availableMemoryProportion,
/// planConstraints and the reduction / load switches pass through;
/// fullyConnectedPass X becomes pass FC_X (NONE: NONE_MATMUL); gatherOutput
/// becomes gatherConvOutput; inputRHSIsPreArranged has no convolution
/// counterpart.
OptionList matMulToConvOptions(const OptionList &matMulOptions);

} // namespace poplin
#endif
