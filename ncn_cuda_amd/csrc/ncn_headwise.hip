// Instantiations and dispatch of the register kernels for heads of one feature (ncn_headwise_kernels.h).
// Compiled four times: as it stands (forward and inverse under the stride permutation); through
// ncn_headwise_bwd.hip (NCN_HEADWISE_BACKWARD = 1: the reversible backward); and each of the two once more
// (ncn_headwise_indexed.hip, ncn_headwise_bwd_indexed.hip: NCN_INDEXED_BUILD = 1) for launches that carry a grouping
// table, a radix level or context lengths.
// The launches come with the geometry of E / w heads of w features (a.head_dim = w = headwise_width(E), a.n_head = E / w).
#include "ncn_configs.h"
#include "ncn_headwise_kernels.h"
#include "ncn_launch.h"

#ifndef NCN_INDEXED_BUILD
#define NCN_INDEXED_BUILD 0
#endif
#ifndef NCN_HEADWISE_BACKWARD
#define NCN_HEADWISE_BACKWARD 0
#endif

namespace ncn {

#if NCN_INDEXED_BUILD && NCN_HEADWISE_BACKWARD
hipError_t launch_headwise_backward_indexed(const StageArgs& a, int grid_x, hipStream_t s) {
#elif NCN_HEADWISE_BACKWARD
hipError_t launch_headwise_backward(const StageArgs& a, int grid_x, hipStream_t s) {
#elif NCN_INDEXED_BUILD
hipError_t launch_headwise_forward_indexed(Pass pass, const StageArgs& a, int grid_x, hipStream_t s) {
#else
hipError_t launch_headwise_forward(Pass pass, const StageArgs& a, int grid_x, hipStream_t s) {
#endif
    constexpr bool kIndexed = NCN_INDEXED_BUILD != 0;
    const dim3 grid(grid_x), block(kBlockThreads);
    const bool tanh_only = a.activation == NCN_ACT_TANH;
#define NCN_LAUNCH(KERNEL) hipLaunchKernelGGL(KERNEL, grid, block, 0, s, a)
#if NCN_HEADWISE_BACKWARD
    // a wave for every tile: the tanh build under the stride permutation has a form without the loop over tiles
    const bool once = !kIndexed && (uint64_t)a.total_tiles * (uint64_t)a.n_head <= (uint64_t)grid_x * kWavesPerBlock;
#define NCN_CASE(NC, EC, R, F)                                                                          \
    if constexpr (EC <= kHeadwiseMaxWidth) {                                                            \
        if (a.n_cache == NC && a.head_dim == EC) {                                                      \
            if (tanh_only && once) NCN_LAUNCH((headwise_backward_kernel<NC, EC, R, F, true, kIndexed, kIndexed>));   \
            else if (tanh_only) NCN_LAUNCH((headwise_backward_kernel<NC, EC, R, F, true, kIndexed>));   \
            else NCN_LAUNCH((headwise_backward_kernel<NC, EC, R, F, false, kIndexed>));                 \
            return hipGetLastError();                                                                   \
        }                                                                                               \
    }
#else
#define NCN_CASE(NC, EC, R, F)                                                                          \
    if constexpr (EC <= kHeadwiseMaxWidth) {                                                            \
        if (a.n_cache == NC && a.head_dim == EC) {                                                      \
            if (pass == kInverse) {                                                                     \
                if (tanh_only) NCN_LAUNCH((headwise_forward_kernel<NC, EC, R, F, true, kIndexed, true>));   \
                else NCN_LAUNCH((headwise_forward_kernel<NC, EC, R, F, false, kIndexed, true>));        \
            } else {                                                                                    \
                if (tanh_only) NCN_LAUNCH((headwise_forward_kernel<NC, EC, R, F, true, kIndexed, false>));  \
                else NCN_LAUNCH((headwise_forward_kernel<NC, EC, R, F, false, kIndexed, false>));       \
            }                                                                                           \
            return hipGetLastError();                                                                   \
        }                                                                                               \
    }
#endif
    NCN_FOR_EACH_FAST_CONFIG(NCN_CASE)
#undef NCN_CASE
#undef NCN_LAUNCH
    return hipErrorInvalidConfiguration;
}

}  // namespace ncn
