// Stand-in for poplar::Target: the device a plan is made for.  This build
// plans for one device only, MI355X (gfx950), so a Target carries nothing a
// plan depends on; it exists so that the tuples poplin::preplan takes
// (include/poplin/Convolution.hpp:386-388 of PopLibs) keep their shape.
#ifndef poplibs_amd_poplar_Target_hpp
#define poplibs_amd_poplar_Target_hpp
#include <string>

namespace poplar {

class Target {
public:
  /// MI355X: 256 compute units in 8 XCDs, 64-lane wavefronts.
  static const Target &gfx950() {
    static const Target target;
    return target;
  }
  unsigned getNumComputeUnits() const { return 256; }
  unsigned getWavefrontSize() const { return 64; }
  std::string getArchitecture() const { return "gfx950"; }
};

} // namespace poplar
#endif
