// bf16-feature instantiations of the destination-row kernel for small graphs, whose long rows are summed by a whole
// workgroup each (rof_coop_kernel; 8 values per lane, fp32 sums, two row gathers in flight).
#include "agg_rows.h"

namespace rofk {

int launch_rows_bf16_coop(const AggArgs &a, const CoopSplit &cs, hipStream_t st) {
    return launch_coop<uint16_t, 8, false>(a, rof_lanes_per_row(a.feat, 8), cs, st);
}

}  // namespace rofk
