// Host-side launch interface between the C ABI (ncn_api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "ncn_device.h"

namespace ncn {

enum Pass { kForward = 0, kInverse = 1, kBackward = 2 };

// Features per lane the register kernels use for (n_cache, head width); 0 = no register kernel.
constexpr int fast_fpl(int nc, int ec) {
    if (!(nc == 2 || nc == 4 || nc == 8 || nc == 16 || nc == 32)) return 0;
    int fpl = 0;
    switch (ec) {
        case 4: fpl = 4; break;
        case 8: fpl = 8; break;
        case 16: fpl = 16; break;
        case 32: fpl = 16; break;
        case 64: fpl = 16; break;
        default: return 0;
    }
    return (nc * (ec / fpl) <= 64) ? fpl : 0;
}

// Groups that one 64-lane wave tile carries on each path.
inline int fast_groups_per_tile(int nc, int ec) { return 64 / (nc * (ec / fast_fpl(nc, ec))); }
inline int generic_groups_per_tile(int nc) { return 64 / nc; }

// Largest head width the generic LDS kernel can hold (7 float arrays of [Ec][64] in 160 KB of LDS).
constexpr int kGenericMaxHeadDim = 64;
constexpr int kGenericArrays = 7;

// Upper bound on gridDim.x of a stage launch == rows of the dW partial buffer.
constexpr int kMaxGridX = 2048;

hipError_t launch_fast_forward(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s);
hipError_t launch_fast_backward(const StageArgs& a, int n_head, int grid_x, hipStream_t s);
hipError_t launch_generic(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s);
hipError_t launch_reduce_dw(const float* partials, int rows, int64_t cols, float* dW, hipStream_t s);

}  // namespace ncn
