// The multi-stage (LDS-resident) passes with one context length per batch entry: the LENGTHS builds of
// ncn_fused_kernels.h, in a translation unit of their own so that they compile beside the plain ones.
#include "ncn_fused_kernels.h"
#include "ncn_fused_pair_kernels.h"
#include "ncn_launch.h"

namespace ncn {

namespace {

template <int NC, int EC>
hipError_t launch_t(Pass pass, const FusedArgs& a, int grid, size_t lds, hipStream_t s) {
    constexpr TileShape t = fast_tile(NC, EC);
    static_assert(t.r != 0, "multi-stage shapes must be one-stage shapes too");
    const bool tanh_only = a.tab.activation == NCN_ACT_TANH;
    hipError_t err;
    if constexpr (NC == 2) {
        if (pass != kBackward && (uint32_t)grid != a.total_items) return hipErrorInvalidConfiguration;
        if (pass == kBackward) {
            const bool loop = (uint32_t)grid < a.total_items;   // see launch_fused_t
            auto k = tanh_only ? (loop ? pair_backward_kernel<EC, true, true, true> : pair_backward_kernel<EC, true, true, false>)
                               : (loop ? pair_backward_kernel<EC, false, true, true> : pair_backward_kernel<EC, false, true, false>);
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kPairWavesBwd), lds, s, a);
        } else if (pass == kInverse) {
            auto k = tanh_only ? pair_forward_kernel<EC, true, true, true> : pair_forward_kernel<EC, false, true, true>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
        } else {
            auto k = tanh_only ? pair_forward_kernel<EC, true, false, true> : pair_forward_kernel<EC, false, false, true>;
            err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
            if (err != hipSuccess) return err;
            hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
        }
        return hipGetLastError();
    } else
    if (pass == kBackward) {
        auto k = tanh_only ? fused_backward_kernel<NC, EC, t.r, t.f, true, false, true>
                           : fused_backward_kernel<NC, EC, t.r, t.f, false, false, true>;
        err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesBwd), lds, s, a);
    } else if (pass == kInverse) {
        auto k = tanh_only ? fused_forward_kernel<NC, EC, t.r, t.f, true, false, true, true>
                           : fused_forward_kernel<NC, EC, t.r, t.f, false, false, true, true>;
        err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
    } else {
        auto k = tanh_only ? fused_forward_kernel<NC, EC, t.r, t.f, true, false, false, true>
                           : fused_forward_kernel<NC, EC, t.r, t.f, false, false, false, true>;
        err = ensure_dynamic_lds(reinterpret_cast<const void*>(k), lds);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(k, dim3(grid), dim3(64 * kFusedWavesFwd), lds, s, a);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_fused_lengths(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s) {
#define NCN_CASE(NC, EC) \
    if (nc == NC && ec == EC) return launch_t<NC, EC>(pass, a, grid, lds, s);
    NCN_FOR_EACH_FUSED_CONFIG(NCN_CASE)
#undef NCN_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace ncn
