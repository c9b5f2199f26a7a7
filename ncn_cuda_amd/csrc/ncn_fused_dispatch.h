// Picks and launches the multi-stage kernel of one pass: shared by the translation units that hold the builds for the
// stride permutation (ncn_fused.hip), context lengths (ncn_fused_lengths.hip), radix levels (ncn_fused_radix.hip) and the
// same three for heads of one feature (ncn_fused_headwise*.hip, ncn_fused_radix_headwise.hip).
#pragma once
#include "ncn_fused_kernels.h"
#include "ncn_fused_pair_kernels.h"
#include "ncn_launch.h"

namespace ncn {

template <int NC, int EC, bool RADIX, bool LENGTHS, bool HEADWISE>
hipError_t launch_fused_build(Pass pass, const FusedArgs& a, int grid, size_t lds, hipStream_t s) {
    constexpr TileShape t = fast_tile(NC, EC);
    static_assert(t.r != 0, "multi-stage shapes must be one-stage shapes too");
    static_assert(!(RADIX && LENGTHS), "context lengths go with the stride permutation");
    const bool backward = pass == kBackward;
    const bool tanh_only = a.tab.activation == NCN_ACT_TANH;
    hipError_t err;
    if constexpr (NC == 2 && !RADIX) {
        static_assert(t.r == 2, "the two-row kernels keep both rows of a group in one lane");
        if (!backward && (uint32_t)grid != a.total_items) return hipErrorInvalidConfiguration;   // one window each
        if (backward) {
            // a workgroup per window when the dW scratch has the rows for it, else workgroups that loop over windows
            const bool loop = (uint32_t)grid < a.total_items;
            auto k = tanh_only ? (loop ? pair_backward_kernel<EC, true, LENGTHS, true, HEADWISE>
                                       : pair_backward_kernel<EC, true, LENGTHS, false, HEADWISE>)
                               : (loop ? pair_backward_kernel<EC, false, LENGTHS, true, HEADWISE>
                                       : pair_backward_kernel<EC, false, LENGTHS, false, HEADWISE>);
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kPairWavesBwd), lds, s, a);
        } else if (pass == kInverse) {
            auto k = tanh_only ? pair_forward_kernel<EC, true, true, LENGTHS, HEADWISE>
                               : pair_forward_kernel<EC, false, true, LENGTHS, HEADWISE>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
        } else {
            auto k = tanh_only ? pair_forward_kernel<EC, true, false, LENGTHS, HEADWISE>
                               : pair_forward_kernel<EC, false, false, LENGTHS, HEADWISE>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
        }
        return hipGetLastError();
    } else {
        if (backward) {
            auto k = tanh_only ? fused_backward_kernel<NC, EC, t.r, t.f, true, RADIX, LENGTHS, HEADWISE>
                               : fused_backward_kernel<NC, EC, t.r, t.f, false, RADIX, LENGTHS, HEADWISE>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesBwd), lds, s, a);
        } else if (pass == kInverse) {
            auto k = tanh_only ? fused_forward_kernel<NC, EC, t.r, t.f, true, RADIX, true, LENGTHS, HEADWISE>
                               : fused_forward_kernel<NC, EC, t.r, t.f, false, RADIX, true, LENGTHS, HEADWISE>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
        } else {
            auto k = tanh_only ? fused_forward_kernel<NC, EC, t.r, t.f, true, RADIX, false, LENGTHS, HEADWISE>
                               : fused_forward_kernel<NC, EC, t.r, t.f, false, RADIX, false, LENGTHS, HEADWISE>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
        }
        return hipGetLastError();
    }
}

// by run-time shape; HEADWISE builds exist for the layouts of up to kHeadwiseMaxWidth adjacent heads
template <bool RADIX, bool LENGTHS, bool HEADWISE>
hipError_t launch_fused_shape(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s) {
#define NCN_CASE(NC, EC)                                                                                  \
    if constexpr (!HEADWISE || EC <= kHeadwiseMaxWidth) {                                                 \
        if (nc == NC && ec == EC) return launch_fused_build<NC, EC, RADIX, LENGTHS, HEADWISE>(pass, a, grid, lds, s); \
    }
    NCN_FOR_EACH_FUSED_CONFIG(NCN_CASE)
#undef NCN_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace ncn
