// fp32-feature instantiations of the row-gather kernel: the partial-sum launches (PHASE 0; PHASE 3 with streaming
// stores of the partial rows; PHASE 5 with more gathers in flight).
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch_partial(const AggArgs &a, int lpr, bool off32, hipStream_t st) {
    return off32 ? launch_lpr<float, 4, PHASE, true, false>(a, lpr, 0, st) : launch_lpr<float, 4, PHASE, false, false>(a, lpr, 0, st);
}

int launch_rows_f32_partial(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec != 4) return launch_lpr<float, 1, 0, false, false>(a, lpr, 0, st);
    if (phase == 5 && off32) return launch_lpr<float, 4, 5, true, false>(a, lpr, 0, st);
    return phase == 3 ? launch_partial<3>(a, lpr, off32, st) : launch_partial<0>(a, lpr, off32, st);
}

}  // namespace rofk
