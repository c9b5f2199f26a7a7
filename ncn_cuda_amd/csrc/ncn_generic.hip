// Generic stage kernels: any n_cache <= 64 and any head width up to kGenericMaxHeadDim, all four
// activations.  One 64-lane wavefront per block, one lane per row, floor(64/n_cache) groups per
// wave tile; the per-row state lives in LDS as [feature][lane] arrays so that the pivot row of a step
// and the sum over a group's rows are plain LDS reads.  This is the slow, shape-agnostic path; the
// register kernels in ncn_stage_kernels.h cover the shapes that matter for speed.
// Same arithmetic as there; see that file for the formulas and their reference citations.
#include <map>
#include <mutex>
#include <utility>

#include "ncn_launch.h"

namespace ncn {

namespace {

struct GenericLane {
    bool valid;
    int64_t off;   // element offset of this lane's row, feature 0 of the head
    int row;       // slot inside the group
    int base;      // lane of slot 0 of this lane's group
    int steps;     // steps of the recurrence = live rows of the group (the same for the whole block)
};

// Wave tile t.  Normal launches: floor(64/n) whole groups, skipping groups a context length cuts.  Edge launches
// (A.edge): t is a batch entry and the tile is its one partly live group, rows and steps = its live rows
// (ncn_triton/ncn_triton_old.py:93-96).
__device__ __forceinline__ GenericLane generic_lane(const StageArgs& A, uint32_t t, int lane, int head) {
    GenericLane L;
    const int n = A.n_cache;
    uint32_t b, group;
    if (A.edge) {
        b = t;
        group = (uint32_t)(live_slots(A, b) / n);
        L.steps = group < A.groups ? live_rows(A, b, group) : 0;
        L.row = lane;
        L.base = 0;
        L.valid = lane < L.steps;
    } else {
        const int gpw = 64 / n;
        const int gw = lane / n;
        L.row = lane - gw * n;
        L.base = gw * n;
        b = t / A.tiles_per_inst;
        const uint32_t tile = t - b * A.tiles_per_inst;
        group = tile * gpw + gw;
        L.steps = n;
        L.valid = (gw < gpw) && (group < A.groups) && live_rows(A, b, group) == n;
    }
    const int64_t pos = slot_position(A, L.valid ? group : 0u, L.valid ? (uint32_t)L.row : 0u);
    L.off = ((int64_t)b * A.N + pos) * A.E + (int64_t)head * A.head_dim;
    if (!L.valid) L.base = lane, L.row = 0;  // idle lanes talk to themselves only
    return L;
}

#define LDS(arr, f) lds[((arr) * ec + (f)) * 64 + lane]
#define LDS_AT(arr, f, l) lds[((arr) * ec + (f)) * 64 + (l)]

// pass 0: forward, pass 1: inverse
__global__ void __launch_bounds__(64) generic_forward_kernel(const StageArgs A, const int inverse) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x, head = blockIdx.y, ec = A.head_dim;
    const float alpha = A.tab.alpha, m = A.tab.m, om = 1.f - A.tab.m, oa = 1.f - A.tab.alpha;
    const float inv_m = 1.f / m, k_ba = om / m;
    const float* Wi = A.W + (int64_t)head * ec;
    const float* Wj = Wi + A.E;
    enum { X = 0, XA = 1 };
    for (uint32_t t = blockIdx.x; t < A.total_tiles; t += gridDim.x) {
        const GenericLane L = generic_lane(A, t, lane, head);
        for (int f = 0; f < ec; ++f) {
            LDS(X, f) = L.valid ? load_elem(A.in0, A.in_dtype, L.off + f) : 0.f;
            LDS(XA, f) = L.valid ? load_elem(A.in1, A.in_dtype, L.off + f) : 0.f;
        }
        __syncthreads();
        for (int step = 0; step < L.steps; ++step) {
            const int j = inverse ? L.steps - 1 - step : step;
            const int jl = L.valid ? L.base + j : lane;
            if (inverse) {
                for (int f = 0; f < ec; ++f) LDS(X, f) = fmaf(LDS(X, f), inv_m, -k_ba * LDS(XA, f));
                __syncthreads();
            }
            float s = 0.f;
            for (int f = 0; f < ec; ++f) s += LDS(X, f) * Wi[f] + LDS_AT(X, f, jl) * Wj[f];
            const float c = oa * s;
            if (inverse) {
                for (int f = 0; f < ec; ++f) {
                    float F, dF;
                    act_fd(A.activation, fmaf(alpha, LDS(X, f), c * LDS_AT(X, f, jl)), F, dF);
                    LDS(XA, f) = fmaf(LDS(XA, f), inv_m, -k_ba * F);
                }
            } else {
                for (int f = 0; f < ec; ++f) {
                    const float xj = LDS_AT(X, f, jl), xv = LDS(X, f);
                    float F, dF;
                    act_fd(A.activation, fmaf(alpha, xv, c * xj), F, dF);
                    const float a2 = fmaf(m, LDS(XA, f), om * F);
                    __syncthreads();  // every lane has read the pivot row's feature f
                    LDS(XA, f) = a2;
                    LDS(X, f) = fmaf(m, xv, om * a2);
                }
            }
            __syncthreads();
        }
        if (L.valid) {
            for (int f = 0; f < ec; ++f) {
                store_elem(A.out0, A.out_dtype, L.off + f, LDS(X, f));
                store_elem(A.out1, A.out_dtype, L.off + f, LDS(XA, f));
                if (A.aux0) {
                    A.aux0[L.off + f] = LDS(X, f);
                    A.aux1[L.off + f] = LDS(XA, f);
                }
            }
        }
        __syncthreads();
    }
}

__global__ void __launch_bounds__(64) generic_backward_kernel(const StageArgs A) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x, head = blockIdx.y, ec = A.head_dim;
    const float alpha = A.tab.alpha, m = A.tab.m, om = 1.f - A.tab.m, oa = 1.f - A.tab.alpha;
    const float inv_m = 1.f / m, k_ba = om / m, k1 = om * om, k2 = om, kh1 = m * om;
    const float* Wi = A.W + (int64_t)head * ec;
    const float* Wj = Wi + A.E;
    enum { X = 0, XA = 1, G = 2, H = 3, U = 4, DWI = 5, DWJ = 6 };
    for (int f = 0; f < ec; ++f) LDS(DWI, f) = LDS(DWJ, f) = 0.f;
    for (uint32_t t = blockIdx.x; t < A.total_tiles; t += gridDim.x) {
        const GenericLane L = generic_lane(A, t, lane, head);
        for (int f = 0; f < ec; ++f) {
            LDS(X, f) = L.valid ? load_elem(A.in0, A.in_dtype, L.off + f) : 0.f;
            LDS(XA, f) = L.valid ? load_elem(A.in1, A.in_dtype, L.off + f) : 0.f;
            LDS(G, f) = L.valid ? load_elem(A.g0, A.g_dtype, L.off + f) : 0.f;
            LDS(H, f) = (L.valid && A.g1) ? load_elem(A.g1, A.g_dtype, L.off + f) : 0.f;
        }
        __syncthreads();
        for (int j = L.steps - 1; j >= 0; --j) {
            const int jl = L.valid ? L.base + j : lane;
            for (int f = 0; f < ec; ++f) LDS(X, f) = fmaf(LDS(X, f), inv_m, -k_ba * LDS(XA, f));
            __syncthreads();
            float s = 0.f;
            for (int f = 0; f < ec; ++f) s += LDS(X, f) * Wi[f] + LDS_AT(X, f, jl) * Wj[f];
            const float c = oa * s;
            float r = 0.f;
            for (int f = 0; f < ec; ++f) {
                const float xj = LDS_AT(X, f, jl);
                float F, dF;
                act_fd(A.activation, fmaf(alpha, LDS(X, f), c * xj), F, dF);
                LDS(XA, f) = fmaf(LDS(XA, f), inv_m, -k_ba * F);
                const float u = fmaf(k1, LDS(G, f), k2 * LDS(H, f)) * dF;
                LDS(U, f) = u;
                r = fmaf(u, xj, r);
            }
            const float cr = oa * r;
            for (int f = 0; f < ec; ++f) {
                const float xj = LDS_AT(X, f, jl), u = LDS(U, f), g = LDS(G, f);
                LDS(DWI, f) = fmaf(r, LDS(X, f), LDS(DWI, f));
                LDS(DWJ, f) = fmaf(r, xj, LDS(DWJ, f));
                LDS(G, f) = fmaf(m, g, fmaf(alpha, u, cr * Wi[f]));
                LDS(H, f) = fmaf(kh1, g, m * LDS(H, f));
                LDS(U, f) = fmaf(cr, Wj[f], c * u);  // this row's share of the pivot row's gradient
            }
            __syncthreads();
            if (L.valid && L.row == j) {
                for (int f = 0; f < ec; ++f) {
                    float v = 0.f;
                    for (int k = 0; k < L.steps; ++k) v += LDS_AT(U, f, L.base + k);
                    LDS(G, f) += v;
                }
            }
            __syncthreads();
        }
        if (L.valid) {
            for (int f = 0; f < ec; ++f) {
                store_elem(A.out0, A.out_dtype, L.off + f, LDS(G, f));
                store_elem(A.out1, A.out_dtype, L.off + f, LDS(H, f));
                if (A.aux0) {
                    A.aux0[L.off + f] = LDS(X, f);
                    A.aux1[L.off + f] = LDS(XA, f);
                }
            }
        }
        __syncthreads();
    }
    // one partial row per block: sum the 64 lanes' accumulators
    for (int k = lane; k < 2 * ec; k += 64) {
        const int half = k / ec, f = k - half * ec;
        float sum = 0.f;
        for (int l = 0; l < 64; ++l) sum += LDS_AT(half ? DWJ : DWI, f, l);
        A.dw_partials[(int64_t)blockIdx.x * (2 * A.E) + (int64_t)half * A.E + (int64_t)head * ec + f] = oa * sum;
    }
}

// dW partial rows are summed in two launches so that the first has enough loads in flight to run at memory speed:
// level 1 sums chunks of kReduceRowsPerBlock rows (block y = one chunk of one segment of the job), level 2 the chunk
// sums of each segment (block y = segment).  A block is 256 / RL columns x RL row lanes (level 2 has few rows of
// blocks, so it takes narrow blocks with many row lanes); the order of additions is fixed.
template <int RL>
__device__ __forceinline__ void reduce_rows(const float* __restrict__ in, int r0, int r1, int64_t row_stride, int64_t cols,
                                            float* __restrict__ out) {
    constexpr int CW = 256 / RL;
    __shared__ float red[RL][CW];
    const int cx = threadIdx.x % CW, ry = threadIdx.x / CW;
    const int64_t col = (int64_t)blockIdx.x * CW + cx;
    float sum = 0.f;
    if (col < cols) {
#pragma unroll 4
        for (int r = r0 + ry; r < r1; r += RL) sum += in[(int64_t)r * row_stride + col];
    }
    red[ry][cx] = sum;
    __syncthreads();
    if (ry == 0 && col < cols) {
        float total = 0.f;
#pragma unroll
        for (int k = 0; k < RL; k += 4) total += (red[k][cx] + red[k + 1][cx]) + (red[k + 2][cx] + red[k + 3][cx]);
        out[col] = total;
    }
}

constexpr int kReduceLevel1Lanes = 4, kReduceLevel2Lanes = 16;

__global__ void __launch_bounds__(256) reduce_chunks_kernel(const ReduceJob J, float* __restrict__ level1) {
    int s = 0;
    while (s + 1 < J.n && (int)blockIdx.y >= J.seg[s + 1].chunk0) ++s;   // at most kReduceMaxSegments - 1 rounds
    const ReduceSegment& g = J.seg[s];
    const int chunk = blockIdx.y - g.chunk0;
    const int r0 = chunk * kReduceRowsPerBlock;
    reduce_rows<kReduceLevel1Lanes>(g.in, r0, min(g.rows, r0 + kReduceRowsPerBlock), g.cols, g.cols,
                                    level1 + g.level1_offset + chunk * g.cols);
}

__global__ void __launch_bounds__(256) reduce_segments_kernel(const ReduceJob J, const float* __restrict__ level1) {
    const ReduceSegment& g = J.seg[blockIdx.y];
    const int chunks = (g.rows + kReduceRowsPerBlock - 1) / kReduceRowsPerBlock;
    reduce_rows<kReduceLevel2Lanes>(level1 + g.level1_offset, 0, chunks, g.cols, g.cols, g.out);
}

// Rows past a batch entry's context length take no part in the stage: they pass through.
//   forward / inverse: out = in (and the float32 copies)     backward: dx = dy, dxa = dya (0 when null), x_rec = y.
// Block (x, y) walks the dead slots live .. N-1 of batch entries y, y + gridDim.y, .., one wavefront per slot.
__global__ void __launch_bounds__(256) pass_through_kernel(const StageArgs A, const int backward, const int64_t batch) {
    const int lane = threadIdx.x & 63;
    for (int64_t bb = blockIdx.y; bb < batch; bb += gridDim.y)
    for (int64_t k = live_slots(A, (uint32_t)bb) + (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); k < A.N;
         k += (int64_t)gridDim.x * 4) {
        const uint32_t b = (uint32_t)bb;
        const int64_t pos = slot_position(A, (uint32_t)(k / A.n_cache), (uint32_t)(k % A.n_cache));
        const int64_t off = ((int64_t)b * A.N + pos) * A.E;
        for (int64_t e = lane; e < A.E; e += 64) {
            const float v0 = load_elem(A.in0, A.in_dtype, off + e, A.plane), v1 = load_elem(A.in1, A.in_dtype, off + e, A.plane);
            if (backward) {
                store_elem(A.out0, A.out_dtype, off + e, load_elem(A.g0, A.g_dtype, off + e));
                store_elem(A.out1, A.out_dtype, off + e, A.g1 ? load_elem(A.g1, A.g_dtype, off + e) : 0.f);
            } else {
                store_elem(A.out0, A.out_dtype, off + e, v0, A.plane);
                store_elem(A.out1, A.out_dtype, off + e, v1, A.plane);
            }
            if (A.aux0) {
                A.aux0[off + e] = v0;
                A.aux1[off + e] = v1;
            }
        }
    }
}

}  // namespace

hipError_t ensure_dynamic_lds(const void* kernel, size_t bytes) {
    static std::mutex mu;
    static std::map<std::pair<int, const void*>, size_t> raised;
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(mu);
    size_t& have = raised[std::make_pair(dev, kernel)];
    if (bytes <= have) return hipSuccess;
    err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (err == hipSuccess) have = bytes;
    return err;
}

hipError_t launch_pass_through(Pass pass, const StageArgs& a, int64_t batch, hipStream_t s) {
    const int64_t per_entry = (a.N + 3) / 4;
    const unsigned gx = (unsigned)(per_entry < 64 ? per_entry : 64);
    const unsigned gy = (unsigned)(batch < 1024 ? batch : 1024);
    hipLaunchKernelGGL(pass_through_kernel, dim3(gx, gy), dim3(256), 0, s, a, pass == kBackward ? 1 : 0, batch);
    return hipGetLastError();
}

hipError_t launch_generic(Pass pass, const StageArgs& a, int n_head, int grid_x, hipStream_t s) {
    const int arrays = (pass == kBackward) ? kGenericArrays : 2;
    const size_t lds_bytes = (size_t)arrays * a.head_dim * 64 * sizeof(float);
    const dim3 grid(grid_x, n_head), block(64);
    hipError_t err;
    if (pass == kBackward) {
        err = ensure_dynamic_lds(reinterpret_cast<const void*>(generic_backward_kernel), lds_bytes);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(generic_backward_kernel, grid, block, lds_bytes, s, a);
    } else {
        err = ensure_dynamic_lds(reinterpret_cast<const void*>(generic_forward_kernel), lds_bytes);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(generic_forward_kernel, grid, block, lds_bytes, s, a, pass == kInverse ? 1 : 0);
    }
    return hipGetLastError();
}

hipError_t launch_reduce_job(const ReduceJob& job, float* level1, hipStream_t s) {
    if (job.n == 0) return hipSuccess;
    int64_t max_cols = 0;
    for (int k = 0; k < job.n; ++k) max_cols = job.seg[k].cols > max_cols ? job.seg[k].cols : max_cols;
    const ReduceSegment& last = job.seg[job.n - 1];
    const int chunks = last.chunk0 + (last.rows + kReduceRowsPerBlock - 1) / kReduceRowsPerBlock;
    constexpr int cw1 = 256 / kReduceLevel1Lanes, cw2 = 256 / kReduceLevel2Lanes;
    hipLaunchKernelGGL(reduce_chunks_kernel, dim3((unsigned)((max_cols + cw1 - 1) / cw1), chunks), dim3(256), 0, s, job,
                       level1);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(reduce_segments_kernel, dim3((unsigned)((max_cols + cw2 - 1) / cw2), job.n), dim3(256), 0, s, job,
                       level1);
    return hipGetLastError();
}

}  // namespace ncn
