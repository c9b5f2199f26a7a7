// A measurement aid, not part of the layer: a kernel that does nothing but independent float32 FMAs, so that a
// benchmark can quote what this GPU sustains on plain (unpacked) v_fma_f32 next to what the NCN kernels reach.
// The library is built without packed FP32 instructions; this kernel is built the same way.
#include <hip/hip_runtime.h>

#include "../../include/ncn_hip.h"

namespace {

constexpr int kChains = 8;   // independent accumulators per lane
constexpr int kUnroll = 8;   // FMAs per accumulator and loop trip

__global__ void __launch_bounds__(256) fma_stream_kernel(float* out, int iters, float b, float c) {
    float a[kChains];
#pragma unroll
    for (int k = 0; k < kChains; ++k) a[k] = b + threadIdx.x * 1e-3f + k;
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
#pragma unroll
            for (int k = 0; k < kChains; ++k) a[k] = fmaf(a[k], b, c);
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < kChains; ++k) s += a[k];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace

extern "C" int ncn_probe_fma_stream(float* out, int blocks, int iters, void* stream) {
    if (!out) return NCN_ERR_NULL;
    if (blocks < 1 || iters < 1) return NCN_ERR_SHAPE;
    hipLaunchKernelGGL(fma_stream_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), out, iters,
                       1.0001f, 0.25f);
    return (int)hipGetLastError();
}

extern "C" int ncn_probe_fma_per_thread(int iters) { return iters > 0 ? iters * kChains * kUnroll : 0; }
