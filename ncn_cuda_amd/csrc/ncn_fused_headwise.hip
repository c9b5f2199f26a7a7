// The multi-stage (LDS-resident) passes for heads of one feature, laid out as heads of 8, 16 or 32 adjacent ones: the
// HEADWISE builds of ncn_fused_kernels.h and ncn_fused_pair_kernels.h under the stride permutation.  Compiled twice: as it
// stands, and through ncn_fused_headwise_lengths.hip (NCN_LENGTHS_BUILD = 1) with a context length per batch entry.
#include "ncn_fused_dispatch.h"

#ifndef NCN_LENGTHS_BUILD
#define NCN_LENGTHS_BUILD 0
#endif

namespace ncn {

#if NCN_LENGTHS_BUILD
hipError_t launch_fused_headwise_lengths(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s) {
    return launch_fused_shape<false, true, true>(pass, a, nc, ec, grid, lds, s);
}
#else
hipError_t launch_fused_headwise(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s) {
    if (a.ctx_len) return launch_fused_headwise_lengths(pass, a, nc, ec, grid, lds, s);
    return launch_fused_shape<false, false, true>(pass, a, nc, ec, grid, lds, s);
}
#endif

}  // namespace ncn
