// fp32-feature instantiations of the row-gather kernel.
#include "agg_rows.h"

namespace rofk {

template <int PHASE, bool CLUSTER>
static int launch_f32(const AggArgs &a, int vec, bool off32, int lds_rows, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 4)
        return off32 ? launch_lpr<float, 4, PHASE, true, CLUSTER>(a, lpr, lds_rows, st)
                     : launch_lpr<float, 4, PHASE, false, CLUSTER>(a, lpr, lds_rows, st);
    return launch_lpr<float, 1, PHASE, false, CLUSTER>(a, lpr, lds_rows, st);
}

int launch_rows_f32(const AggArgs &a, int phase, int vec, bool off32, int lds_rows, hipStream_t st) {
    if (phase == 0) return launch_f32<0, false>(a, vec, off32, 0, st);
    if (lds_rows > 0) return phase == 1 ? launch_f32<1, true>(a, vec, off32, lds_rows, st) : launch_f32<2, true>(a, vec, off32, lds_rows, st);
    return phase == 1 ? launch_f32<1, false>(a, vec, off32, 0, st) : launch_f32<2, false>(a, vec, off32, 0, st);
}

}  // namespace rofk
