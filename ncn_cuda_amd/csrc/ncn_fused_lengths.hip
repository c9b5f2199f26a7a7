// The multi-stage (LDS-resident) passes with one context length per batch entry: the LENGTHS builds of
// ncn_fused_kernels.h, in a translation unit of their own so that they compile beside the plain ones.
#include "ncn_fused_dispatch.h"

namespace ncn {

hipError_t launch_fused_lengths(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s) {
    return launch_fused_shape<false, true, false>(pass, a, nc, ec, grid, lds, s);
}

}  // namespace ncn
