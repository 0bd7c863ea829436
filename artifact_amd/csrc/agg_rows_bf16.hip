// bf16-feature (fp32-accumulate) instantiations of the row-gather kernel.
#include "agg_rows.h"

namespace rofk {

template <int PHASE>
static int launch_bf16(const AggArgs &a, int vec, bool off32, hipStream_t st) {
    const int lpr = rof_lanes_per_row(a.feat, vec);
    if (vec == 8)
        return off32 ? launch_lpr<uint16_t, 8, PHASE, true>(a, lpr, st)
                     : launch_lpr<uint16_t, 8, PHASE, false>(a, lpr, st);
    return launch_lpr<uint16_t, 1, PHASE, false>(a, lpr, st);
}

int launch_rows_bf16(const AggArgs &a, int phase, int vec, bool off32, hipStream_t st) {
    if (phase == 0) return launch_bf16<0>(a, vec, off32, st);
    return phase == 1 ? launch_bf16<1>(a, vec, off32, st) : launch_bf16<2>(a, vec, off32, st);
}

}  // namespace rofk
