// fp32-feature instantiations of the row-gather kernel: the destination-row launch (PHASE 1; PHASE 2 with streaming
// stores; PHASE 4 with more gathers in flight).
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch(const AggArgs &a, int vec, bool off32, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 4)
        return off32 ? launch_lpr<float, 4, PHASE, true, false>(a, lpr, 0, st)
                     : launch_lpr<float, 4, PHASE, false, false>(a, lpr, 0, st);
    return launch_lpr<float, 1, PHASE, false, false>(a, lpr, 0, st);
}

int launch_rows_f32_dst(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st) {
    if (phase == 4 && vec == 4 && off32) return launch_lpr<float, 4, 4, true, false>(a, rof_lanes_per_row(a.feat, vec), 0, st);
    return phase == 2 ? launch<2>(a, vec, off32, st) : launch<1>(a, vec, off32, st);
}

}  // namespace rofk
