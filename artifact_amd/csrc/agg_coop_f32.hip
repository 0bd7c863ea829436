// fp32-feature instantiations of the destination-row kernel for small graphs, whose long rows are summed by a whole
// workgroup each (rof_coop_kernel), with two or with four row gathers in flight.
#include "agg_rows.h"

namespace rofk {

int launch_rows_f32_coop(const AggArgs &a, bool deep, const CoopSplit &cs, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, 4);
    return deep ? launch_coop<float, 4, true>(a, lpr, cs, st) : launch_coop<float, 4, false>(a, lpr, cs, st);
}

}  // namespace rofk
