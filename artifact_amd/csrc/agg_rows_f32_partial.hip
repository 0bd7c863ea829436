// fp32-feature instantiations of the row-gather kernel: the partial-sum launches (PHASE 0).
#include "agg_rows.h"

namespace rofk {

int launch_rows_f32_partial(const AggArgs &a, int vec, bool off32, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 4)
        return off32 ? launch_lpr<float, 4, 0, true, false>(a, lpr, 0, st) : launch_lpr<float, 4, 0, false, false>(a, lpr, 0, st);
    return launch_lpr<float, 1, 0, false, false>(a, lpr, 0, st);
}

}  // namespace rofk
