// bf16-feature instantiations of the row-gather kernel: the partial-sum launches (PHASE 0, and PHASE 3 with
// streaming stores of the partial rows).
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch_partial(const AggArgs &a, int lpr, bool off32, hipStream_t st) {
    return off32 ? launch_lpr<uint16_t, 8, PHASE, true, false>(a, lpr, 0, st) : launch_lpr<uint16_t, 8, PHASE, false, false>(a, lpr, 0, st);
}

int launch_rows_bf16_partial(const AggArgs &a, bool stream, int vec, bool off32, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 8) return stream ? launch_partial<3>(a, lpr, off32, st) : launch_partial<0>(a, lpr, off32, st);
    return launch_lpr<uint16_t, 1, 0, false, false>(a, lpr, 0, st);
}

}  // namespace rofk
