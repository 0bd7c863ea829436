// fp32-feature instantiations of the row-gather kernel: the clustered destination rows (rof_cluster_kernel).
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch(const AggArgs &a, int vec, bool off32, int lds_rows, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 4)
        return off32 ? launch_lpr<float, 4, PHASE, true, true>(a, lpr, lds_rows, st)
                     : launch_lpr<float, 4, PHASE, false, true>(a, lpr, lds_rows, st);
    return launch_lpr<float, 1, PHASE, false, true>(a, lpr, lds_rows, st);
}

int launch_rows_f32_cluster(const AggArgs &a, int phase, int vec, bool off32, int lds_rows, hipStream_t st) {
    return phase == 1 ? launch<1>(a, vec, off32, lds_rows, st) : launch<2>(a, vec, off32, lds_rows, st);
}

}  // namespace rofk
