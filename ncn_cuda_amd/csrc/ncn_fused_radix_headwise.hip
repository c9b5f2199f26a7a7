// The multi-stage passes over radix-n levels for heads of one feature: the RADIX, HEADWISE builds of
// ncn_fused_kernels.h (planning and geometry: ncn_fused_radix.hip).
#include "ncn_fused_dispatch.h"

namespace ncn {

hipError_t launch_fused_radix_headwise(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s) {
    return launch_fused_shape<true, false, true>(pass, a, nc, ec, grid, lds, s);
}

}  // namespace ncn
