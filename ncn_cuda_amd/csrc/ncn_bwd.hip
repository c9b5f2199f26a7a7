// Instantiations and dispatch of the register-resident reversible backward stage kernel.
// Compiled four times: as it stands for the stride permutation; through ncn_bwd_indexed.hip (NCN_INDEXED_BUILD = 1)
// for launches that carry a grouping table or context lengths; and each of the two once more (ncn_bwd_once.hip,
// ncn_bwd_indexed_once.hip: NCN_ONCE_BUILD = 1) in the form without a loop over tiles, which the launchers pick by
// themselves when the grid has a wave for every tile.
#include "ncn_configs.h"
#include "ncn_launch.h"
#include "ncn_stage_kernels.h"

#ifndef NCN_INDEXED_BUILD
#define NCN_INDEXED_BUILD 0
#endif
#ifndef NCN_ONCE_BUILD
#define NCN_ONCE_BUILD 0
#endif

namespace ncn {

#if NCN_INDEXED_BUILD && NCN_ONCE_BUILD
hipError_t launch_fast_backward_indexed_once(const StageArgs& a, int /*n_head*/, int grid_x, hipStream_t s) {
#elif NCN_INDEXED_BUILD
hipError_t launch_fast_backward_indexed(const StageArgs& a, int n_head, int grid_x, hipStream_t s) {
    if ((uint64_t)a.total_tiles * (uint64_t)a.n_head <= (uint64_t)grid_x * kWavesPerBlock)
        return launch_fast_backward_indexed_once(a, n_head, grid_x, s);   // a wave for every tile
#elif NCN_ONCE_BUILD
hipError_t launch_fast_backward_once(const StageArgs& a, int /*n_head*/, int grid_x, hipStream_t s) {
#else
hipError_t launch_fast_backward(const StageArgs& a, int n_head, int grid_x, hipStream_t s) {
    if ((uint64_t)a.total_tiles * (uint64_t)a.n_head <= (uint64_t)grid_x * kWavesPerBlock)
        return launch_fast_backward_once(a, n_head, grid_x, s);   // a wave for every tile
#endif
    constexpr bool kIndexed = NCN_INDEXED_BUILD != 0;
    constexpr bool kLoop = NCN_ONCE_BUILD == 0;
    const dim3 grid(grid_x), block(kBlockThreads);
    const bool tanh_only = a.activation == NCN_ACT_TANH;
#define NCN_CASE(NC, EC, R, F)                                                                  \
    static_assert(fast_tile(NC, EC).r == R && fast_tile(NC, EC).f == F, "duplicate config entry");          \
    if (a.n_cache == NC && a.head_dim == EC) {                                                 \
        if (tanh_only) hipLaunchKernelGGL((stage_backward_kernel<NC, EC, R, F, true, kIndexed, kLoop>), grid, block, 0, s, a); \
        else hipLaunchKernelGGL((stage_backward_kernel<NC, EC, R, F, false, kIndexed, kLoop>), grid, block, 0, s, a);          \
        return hipGetLastError();                                                              \
    }
    NCN_FOR_EACH_FAST_CONFIG(NCN_CASE)
#undef NCN_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace ncn
