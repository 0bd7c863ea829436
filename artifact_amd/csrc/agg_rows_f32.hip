// fp32-feature instantiations of the row-gather kernel.
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch_f32(const AggArgs &a, int vec, bool off32, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 4)
        return off32 ? launch_lpr<float, 4, PHASE, true>(a, lpr, st) : launch_lpr<float, 4, PHASE, false>(a, lpr, st);
    return launch_lpr<float, 1, PHASE, false>(a, lpr, st);
}

int launch_rows_f32(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st) {
    if (phase == 0) return launch_f32<0>(a, vec, off32, st);
    return phase == 1 ? launch_f32<1>(a, vec, off32, st) : launch_f32<2>(a, vec, off32, st);
}

}  // namespace rofk
