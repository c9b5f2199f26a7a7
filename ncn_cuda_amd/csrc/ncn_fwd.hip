// Instantiations and dispatch of the register-resident forward and inverse stage kernels.
#include "ncn_configs.h"
#include "ncn_launch.h"
#include "ncn_stage_kernels.h"

namespace ncn {

hipError_t launch_fast_forward(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s) {
    const dim3 grid(grid_x), block(kBlockThreads);
    const bool tanh_only = a.activation == NCN_ACT_TANH;
#define NCN_CASE(NC, EC, R, F)                                                                        \
    static_assert(fast_tile(NC, EC).r == R && fast_tile(NC, EC).f == F, "duplicate config entry");                \
    if (a.n_cache == NC && a.head_dim == EC) {                                                       \
        if (pass == kInverse) {                                                                      \
            if (tanh_only) hipLaunchKernelGGL((stage_inverse_kernel<NC, EC, R, F, true>), grid, block, 0, s, a); \
            else hipLaunchKernelGGL((stage_inverse_kernel<NC, EC, R, F, false>), grid, block, 0, s, a);          \
        } else {                                                                                     \
            if (tanh_only) hipLaunchKernelGGL((stage_forward_kernel<NC, EC, R, F, true>), grid, block, 0, s, a); \
            else hipLaunchKernelGGL((stage_forward_kernel<NC, EC, R, F, false>), grid, block, 0, s, a);          \
        }                                                                                            \
        return hipGetLastError();                                                                    \
    }
    NCN_FOR_EACH_FAST_CONFIG(NCN_CASE)
#undef NCN_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace ncn
