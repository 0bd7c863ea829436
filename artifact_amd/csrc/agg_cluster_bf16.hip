// bf16-feature instantiations of the row-gather kernel: the clustered destination rows (rof_cluster_kernel).
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch(const AggArgs &a, int vec, bool off32, int lds_rows, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 8)
        return off32 ? launch_lpr<uint16_t, 8, PHASE, true, true>(a, lpr, lds_rows, st)
                     : launch_lpr<uint16_t, 8, PHASE, false, true>(a, lpr, lds_rows, st);
    return launch_lpr<uint16_t, 1, PHASE, false, true>(a, lpr, lds_rows, st);
}

int launch_rows_bf16_cluster(const AggArgs &a, int phase, int vec, bool off32, int lds_rows, hipStream_t st) {
    return phase == 1 ? launch<1>(a, vec, off32, lds_rows, st) : launch<2>(a, vec, off32, lds_rows, st);
}

}  // namespace rofk
