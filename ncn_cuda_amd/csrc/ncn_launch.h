// Host-side launch interface between the C ABI (ncn_api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <vector>

#include "ncn_configs.h"
#include "ncn_device.h"

namespace ncn {

enum Pass { kForward = 0, kInverse = 1, kBackward = 2 };

// Register tile (rows x features per lane) the register kernels use for (n_cache, head width); {0,0} = none.
struct TileShape {
    int r, f;
};
constexpr TileShape fast_tile(int nc, int ec) {
#define NCN_MATCH(NC, EC, R, F) \
    if (nc == NC && ec == EC) return TileShape{R, F};
    NCN_FOR_EACH_FAST_CONFIG(NCN_MATCH)
#undef NCN_MATCH
    return TileShape{0, 0};
}

// Groups that one 64-lane wave tile carries on each path.
inline int fast_groups_per_tile(int nc, int ec) {
    const TileShape t = fast_tile(nc, ec);
    return 64 / ((nc / t.r) * (ec / t.f));
}
inline int generic_groups_per_tile(int nc) { return 64 / nc; }

// Largest head width the generic LDS kernel can hold (7 float arrays of [Ec][64] in 160 KB of LDS).
constexpr int kGenericMaxHeadDim = 64;
constexpr int kGenericArrays = 7;

// Upper bound on gridDim.x of a stage launch == rows of the dW partial buffer.
constexpr int kMaxGridX = 16384;
// Upper bound on gridDim.x of a forward / inverse launch (no partial rows to pay for).
constexpr int kMaxForwardGridX = 1 << 18;
// dW partial rows are summed in two levels: chunks of kReduceRowsPerBlock rows, then the chunk sums.
constexpr int kReduceRowsPerBlock = 32;
// One reduction job sums up to kReduceMaxSegments partial arrays (one per backward launch of a call) that lie side by
// side in the partial buffer and hold at most kReduceMaxStages stages between them.
constexpr int kReduceMaxSegments = 8;
constexpr int kReduceMaxStages = 8;
// Rows of 2E floats that level 1 may need: sum over segments of ceil(rows / 32) * stages, where the segments' rows *
// stages add up to at most kMaxGridX and their stages to at most kReduceMaxStages.
constexpr int kReduceLevel1Rows = kMaxGridX / kReduceRowsPerBlock + kReduceMaxStages;
struct ReduceSegment {
    const float* in;        // [rows][cols], dense
    float* out;             // [cols]
    int64_t cols;           // stages of the launch * 2E
    int64_t level1_offset;  // floats before this segment's chunk sums in the level-1 scratch
    int rows;
    int chunk0;             // chunks of the segments before this one
};
struct ReduceJob {
    ReduceSegment seg[kReduceMaxSegments];
    int n;
};
// out[col] of every segment = sum of its rows, in a fixed order; level1 is scratch of kReduceLevel1Rows * 2E floats.
hipError_t launch_reduce_job(const ReduceJob& job, float* level1, hipStream_t s);

// Raises a kernel's dynamic LDS limit to `bytes` on the current device unless an earlier call already raised it that
// far (the limit is kept per device and kernel for the life of the process: one driver call instead of one per launch).
hipError_t ensure_dynamic_lds(const void* kernel, size_t bytes);

hipError_t launch_fast_forward(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s);
hipError_t launch_fast_backward(const StageArgs& a, int n_head, int grid_x, hipStream_t s);
// the same for a grid that has a wave for every tile (ncn_bwd_once.hip); launch_fast_backward goes there by itself
hipError_t launch_fast_backward_once(const StageArgs& a, int n_head, int grid_x, hipStream_t s);
// the same kernels built to honour a.table and a.ctx_len (the plain builds ignore both)
hipError_t launch_fast_forward_indexed(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s);
hipError_t launch_fast_backward_indexed(const StageArgs& a, int n_head, int grid_x, hipStream_t s);
hipError_t launch_fast_backward_indexed_once(const StageArgs& a, int n_head, int grid_x, hipStream_t s);
// Heads of one feature (ncn_headwise_kernels.h): `a` carries the geometry of E / w heads of w features, w =
// headwise_width(E), for which the grid was planned as well; the second form honours a.table, a.radix_stride and
// a.ctx_len.
constexpr int kHeadwiseMaxWidth = 32;
// adjacent one-feature heads that the lanes of a row hold together: the largest of 32, 16, 8, 4 that divides E (0: none)
constexpr int headwise_width(int64_t E) {
    for (int w = kHeadwiseMaxWidth; w >= 4; w /= 2)
        if (E % w == 0) return w;
    return 0;
}
hipError_t launch_headwise_forward(Pass pass, const StageArgs& a, int grid_x, hipStream_t s);
hipError_t launch_headwise_forward_indexed(Pass pass, const StageArgs& a, int grid_x, hipStream_t s);
hipError_t launch_headwise_backward(const StageArgs& a, int grid_x, hipStream_t s);
hipError_t launch_headwise_backward_indexed(const StageArgs& a, int grid_x, hipStream_t s);
hipError_t launch_generic(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s);
// Rows past the context length of their batch entry: copied through (a.ctx_len must be set).
hipError_t launch_pass_through(Pass pass, const StageArgs& a, int64_t batch, hipStream_t s);
// gridDim.x of the generic kernel's edge launch (the partly live group of each batch entry) == its dW partial rows.
constexpr int kEdgeGridX = 256;
// ---- multi-stage (LDS-resident) passes, ncn_fused.hip --------------------------------------------------------
struct FusedArgs;
struct FusedPass {
    int first, count;  // stages [first, first + count) relative to the range that was planned
    int single;        // 1: not worth fusing, run `first` with the one-stage kernel
    uint32_t class_stride, ring, window, halo, own, tiles_per_ring, closed, class_groups;
    uint32_t sub_stride[8];
};
bool fused_supported(const ncn_shape* sh, int activation);
std::vector<FusedPass> plan_fused(const ncn_shape* sh, int first, int count, bool backward);
// windows of a pass (== workgroups, when every workgroup takes one)
int64_t fused_items(const ncn_shape* sh, const FusedPass& p);
// row_cap: rows of the dW partial buffer a backward pass may fill (grid / n_head rows per stage)
int fused_grid(const ncn_shape* sh, const FusedPass& p, bool backward, int row_cap = kMaxGridX);
// headwise: `sh` is the layout of a call on heads of one feature (headwise_width(E) adjacent heads to a "head")
hipError_t launch_fused(Pass pass, FusedArgs& a, const ncn_shape* sh, const FusedPass& p, hipStream_t s,
                        int row_cap = kMaxGridX, bool headwise = false);
// the builds with context lengths (a.ctx_len set), ncn_fused_lengths.hip; launch_fused goes there by itself
hipError_t launch_fused_lengths(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s);
// the builds for heads of one feature (ncn_fused_headwise.hip; the first goes to the second when a.ctx_len is set)
hipError_t launch_fused_headwise(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s);
hipError_t launch_fused_headwise_lengths(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s);


// ---- multi-stage passes over radix-n levels, ncn_fused_radix.hip ---------------------------------------------
struct RadixPass {
    int first, count;  // levels [first, first + count) relative to the range that was planned
    int single;        // 1: one level, run with the one-stage kernel
    uint32_t s0;       // n^(first level of the pass): distance in rows between the rows of a window
    uint32_t span;     // n^count: rows of a window
    uint32_t rows;     // rows a workgroup holds (a whole number of windows)
    uint32_t loads;    // workgroup-loads per batch entry and head
};
bool radix_fused_supported(const ncn_shape* sh);
// fused = false: one level per pass whatever the shape (calls whose scalars only the generic kernels take)
std::vector<RadixPass> plan_radix(const ncn_shape* sh, int first, int count, bool backward, bool fused = true);
int radix_grid(const ncn_shape* sh, const RadixPass& p, bool backward);
hipError_t launch_fused_radix(Pass pass, FusedArgs& a, const ncn_shape* sh, const RadixPass& p, hipStream_t s,
                              bool headwise = false);
hipError_t launch_fused_radix_headwise(Pass pass, const FusedArgs& a, int nc, int ec, int grid, size_t lds, hipStream_t s);

}  // namespace ncn
