// poplin::preplan (include/poplin/ConvPreplan.hpp:36-37 of PopLibs): plan a
// set of convolutions and matrix multiplications ahead of use and leave the
// plans in a PlanningCache, so that the first convolution() / matMul() of each
// finds its plan there.
#ifndef poplibs_amd_poplin_ConvPreplan_hpp
#define poplibs_amd_poplin_ConvPreplan_hpp
#include "poplin/Convolution.hpp"
#include "poplin/MatMul.hpp"

#include <set>

namespace poplin {

/// Plans every entry of `convs` and `matmuls` (the entries' Target pointers
/// may be null: this build plans for MI355X only) and adds the plans to
/// `cache`.  The plans are made on several host threads and inserted one
/// after the other, as the reference does with TBB
/// (lib/poplin/ConvPlan.cpp:1839-1875).  An entry whose parameters or options
/// are invalid throws what planning it alone would, after which `cache` holds
/// none of this call's plans.
void preplan(const std::set<ConvPlanParams> &convs,
             const std::set<MatMulPlanParams> &matmuls, PlanningCache &cache);

/// The older name for planning convolutions only
/// (include/poplin/Convolution.hpp:386-401 of PopLibs, deprecated there in
/// favour of preplan).
void preplanConvolutions(const std::set<ConvPlanParams> &convs,
                         PlanningCache &cache);

} // namespace poplin
#endif
