// Register-resident stage kernels: forward, inverse and reversible backward of ONE stage.
//
// Work decomposition.  A (batch, head, group) triple is an independent problem: n_cache rows of Ec
// features (torch_ref/ncn_pytorch.py:50-97).  A row is split over LPR = Ec/FPL adjacent lanes that each
// keep FPL features of x and xa (and of the two gradients) in registers; the n_cache rows of a group
// occupy n_cache*LPR adjacent lanes, so one 64-wide wavefront carries 64/(n_cache*LPR) whole groups
// ("a wave tile") and no step of the recurrence ever needs a workgroup barrier:
//   * the pivot row x_j of a step reaches the other rows with one ds_bpermute per register,
//   * <x_i,Wi> + <x_j,Wj> and <u_i,x_j> are in-lane FMAs plus log2(LPR) cross-lane adds,
//   * the sum over rows that feeds the pivot row's gradient is log2(n_cache) cross-lane adds.
// A wave loops over wave tiles of one head (blockIdx.y), keeps that head's slices of Wi, Wj in
// registers, and in backward accumulates dWi, dWj in registers over all its tiles; they are reduced
// across lanes and waves once per block and leave as one [2*Ec] partial per block.
//
// Memory: a lane reads and writes only its own FPL-feature fragment of its own row (16-byte vector
// accesses; a row of one head is one contiguous Ec*4-byte segment), each row exactly once per stage.
#pragma once
#include "ncn_device.h"

namespace ncn {

constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = 64 * kWavesPerBlock;

template <int NC, int EC, int FPL>
struct Tile {
    static_assert(EC % FPL == 0, "FPL must divide the head width");
    static constexpr int LPR = EC / FPL;       // lanes per row
    static constexpr int LPG = NC * LPR;       // lanes per group
    static_assert(LPG <= 64 && 64 % LPG == 0, "a group must fit one wavefront");
    static constexpr int GPW = 64 / LPG;       // groups per wave tile
    static constexpr int ROWMASK = (NC - 1) * LPR;
};

// Position of this lane's row and validity, for wave tile `t`.
template <int NC, int EC, int FPL>
__device__ __forceinline__ bool tile_row_offset(const StageArgs& A, uint32_t t, int lane, int head, int64_t& off) {
    using T = Tile<NC, EC, FPL>;
    const int q = lane % T::LPR;
    const int i = (lane / T::LPR) % NC;
    const int gw = lane / T::LPG;
    const uint32_t b = t / A.tiles_per_inst;
    const uint32_t tile = t - b * A.tiles_per_inst;
    const uint32_t group = tile * T::GPW + gw;
    const bool valid = group < A.groups;
    const uint32_t blk = stage_block(A, valid ? group : 0u, (uint32_t)i);
    const int64_t pos = (int64_t)blk * NC + i;
    off = ((int64_t)b * A.N + pos) * A.E + (int64_t)head * EC + q * FPL;
    return valid;
}

template <int FPL>
__device__ __forceinline__ void load_w(const StageArgs& A, int head, int ec, int q, float (&wi)[FPL], float (&wj)[FPL]) {
    const float* w = A.W + (int64_t)head * ec + q * FPL;
#pragma unroll
    for (int f = 0; f < FPL; ++f) {
        wi[f] = w[f];
        wj[f] = w[A.E + f];
    }
}

// ---------------------------------------------------------------------------------------------
// forward (torch_ref/ncn_pytorch.py:74-94)
// ---------------------------------------------------------------------------------------------
template <int NC, int EC, int FPL>
__global__ void __launch_bounds__(kBlockThreads) stage_forward_kernel(const StageArgs A) {
    using T = Tile<NC, EC, FPL>;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int head = blockIdx.y;
    const int q = lane % T::LPR;
    const float alpha = A.alpha, m = A.m, om = 1.0f - A.m, oa = 1.0f - A.alpha;

    float wi[FPL], wj[FPL];
    load_w<FPL>(A, head, EC, q, wi, wj);

    const uint32_t nwaves = gridDim.x * kWavesPerBlock;
    for (uint32_t t = blockIdx.x * kWavesPerBlock + wave; t < A.total_tiles; t += nwaves) {
        int64_t off;
        const bool valid = tile_row_offset<NC, EC, FPL>(A, t, lane, head, off);
        float x[FPL], a[FPL];
        load_frag<FPL>(A.in0, A.in_dtype, off, valid, x);
        load_frag<FPL>(A.in1, A.in_dtype, off, valid, a);

#pragma unroll 1
        for (int j = 0; j < NC; ++j) {
            const int src = (lane & ~T::ROWMASK) | (j * T::LPR);
            float xj[FPL];
            float d = 0.f, e = 0.f;
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                xj[f] = lane_read(x[f], src);
                d = fmaf(x[f], wi[f], d);
                e = fmaf(xj[f], wj[f], e);
            }
            const float s = lane_sum<1, T::LPR>(d + e);
            const float c = oa * s;
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                const float Tv = fmaf(alpha, x[f], c * xj[f]);
                const float F = tanh_f(Tv);
                a[f] = fmaf(m, a[f], om * F);
                x[f] = fmaf(m, x[f], om * a[f]);
            }
        }
        store_frag<FPL>(A.out0, A.out_dtype, off, valid, x);
        store_frag<FPL>(A.out1, A.out_dtype, off, valid, a);
        if (A.aux0) {
            store_frag<FPL>(A.aux0, NCN_F32, off, valid, x);
            store_frag<FPL>(A.aux1, NCN_F32, off, valid, a);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// inverse (torch_ref/ncn_pytorch_invertible.py:87-113), steps j = n_cache-1 .. 0
// ---------------------------------------------------------------------------------------------
template <int NC, int EC, int FPL>
__global__ void __launch_bounds__(kBlockThreads) stage_inverse_kernel(const StageArgs A) {
    using T = Tile<NC, EC, FPL>;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int head = blockIdx.y;
    const int q = lane % T::LPR;
    const float alpha = A.alpha, oa = 1.0f - A.alpha;
    const float inv_m = 1.0f / A.m, k_ba = (1.0f - A.m) / A.m;

    float wi[FPL], wj[FPL];
    load_w<FPL>(A, head, EC, q, wi, wj);

    const uint32_t nwaves = gridDim.x * kWavesPerBlock;
    for (uint32_t t = blockIdx.x * kWavesPerBlock + wave; t < A.total_tiles; t += nwaves) {
        int64_t off;
        const bool valid = tile_row_offset<NC, EC, FPL>(A, t, lane, head, off);
        float y[FPL], b[FPL];
        load_frag<FPL>(A.in0, A.in_dtype, off, valid, y);
        load_frag<FPL>(A.in1, A.in_dtype, off, valid, b);

#pragma unroll 1
        for (int j = NC - 1; j >= 0; --j) {
            const int src = (lane & ~T::ROWMASK) | (j * T::LPR);
            float xj[FPL];
            float d = 0.f, e = 0.f;
#pragma unroll
            for (int f = 0; f < FPL; ++f) y[f] = fmaf(y[f], inv_m, -k_ba * b[f]);  // x of this step
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                xj[f] = lane_read(y[f], src);
                d = fmaf(y[f], wi[f], d);
                e = fmaf(xj[f], wj[f], e);
            }
            const float s = lane_sum<1, T::LPR>(d + e);
            const float c = oa * s;
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                const float Tv = fmaf(alpha, y[f], c * xj[f]);
                const float F = tanh_f(Tv);
                b[f] = fmaf(b[f], inv_m, -k_ba * F);  // xa of this step
            }
        }
        store_frag<FPL>(A.out0, A.out_dtype, off, valid, y);
        store_frag<FPL>(A.out1, A.out_dtype, off, valid, b);
    }
}

// ---------------------------------------------------------------------------------------------
// reversible backward: per step, invert (ncn_bwd_cuda_kernel.cu:88-115), then the closed-form
// vector-Jacobian product (the vectorised statement is ncn_triton/ncn_triton.py:198-246):
//   q = (1-m)^2 g + (1-m) h      u = q * F'(T)       r_i = <u_i, x_j>
//   dWi += (1-a) r_i x_i         dWj += (1-a) r_i x_j
//   g_i <- m g_i + a u_i + (1-a) r_i Wi  [+ sum_k ((1-a) r_k Wj + (1-a) s_k u_k) on the pivot row]
//   h_i <- m (1-m) g_i + m h_i
// ---------------------------------------------------------------------------------------------
template <int NC, int EC, int FPL>
__global__ void __launch_bounds__(kBlockThreads) stage_backward_kernel(const StageArgs A) {
    using T = Tile<NC, EC, FPL>;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int head = blockIdx.y;
    const int q = lane % T::LPR;
    const int row = (lane / T::LPR) % NC;
    const float alpha = A.alpha, m = A.m, om = 1.0f - A.m, oa = 1.0f - A.alpha;
    const float inv_m = 1.0f / m, k_ba = om / m;
    const float k1 = om * om, k2 = om, kh1 = m * om;

    float wi[FPL], wj[FPL];
    load_w<FPL>(A, head, EC, q, wi, wj);
    float dwi[FPL], dwj[FPL];
#pragma unroll
    for (int f = 0; f < FPL; ++f) dwi[f] = dwj[f] = 0.f;

    const uint32_t nwaves = gridDim.x * kWavesPerBlock;
    for (uint32_t t = blockIdx.x * kWavesPerBlock + wave; t < A.total_tiles; t += nwaves) {
        int64_t off;
        const bool valid = tile_row_offset<NC, EC, FPL>(A, t, lane, head, off);
        float y[FPL], b[FPL], g[FPL], h[FPL];
        load_frag<FPL>(A.in0, A.in_dtype, off, valid, y);
        load_frag<FPL>(A.in1, A.in_dtype, off, valid, b);
        load_frag<FPL>(A.g0, A.g_dtype, off, valid, g);
        load_frag<FPL>(A.g1, A.g_dtype, off, valid && A.g1 != nullptr, h);

#pragma unroll 1
        for (int j = NC - 1; j >= 0; --j) {
            const int src = (lane & ~T::ROWMASK) | (j * T::LPR);
            float xj[FPL], u[FPL];
            float d = 0.f, e = 0.f;
#pragma unroll
            for (int f = 0; f < FPL; ++f) y[f] = fmaf(y[f], inv_m, -k_ba * b[f]);  // x of this step
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                xj[f] = lane_read(y[f], src);
                d = fmaf(y[f], wi[f], d);
                e = fmaf(xj[f], wj[f], e);
            }
            const float s = lane_sum<1, T::LPR>(d + e);
            const float c = oa * s;
            float r = 0.f;
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                const float Tv = fmaf(alpha, y[f], c * xj[f]);
                float F, dF;
                tanh_fd(Tv, F, dF);
                b[f] = fmaf(b[f], inv_m, -k_ba * F);  // xa of this step
                const float qq = fmaf(k1, g[f], k2 * h[f]);
                u[f] = qq * dF;
                r = fmaf(u[f], xj[f], r);
            }
            r = lane_sum<1, T::LPR>(r);
            const float cr = oa * r;
            const bool pivot = (row == j);
#pragma unroll
            for (int f = 0; f < FPL; ++f) {
                dwi[f] = fmaf(r, y[f], dwi[f]);
                dwj[f] = fmaf(r, xj[f], dwj[f]);
                float v = fmaf(cr, wj[f], c * u[f]);
                v = lane_sum<T::LPR, T::LPG>(v);  // over the rows of the group
                const float gn = fmaf(m, g[f], fmaf(alpha, u[f], cr * wi[f]));
                h[f] = fmaf(kh1, g[f], m * h[f]);
                g[f] = pivot ? gn + v : gn;
            }
        }
        store_frag<FPL>(A.out0, A.out_dtype, off, valid, g);
        store_frag<FPL>(A.out1, A.out_dtype, off, valid, h);
        if (A.aux0) {
            store_frag<FPL>(A.aux0, NCN_F32, off, valid, y);
            store_frag<FPL>(A.aux1, NCN_F32, off, valid, b);
        }
    }

    // dW: lanes holding the same feature chunk q -> one value; then across the block's waves.
    __shared__ float red[kWavesPerBlock][2][EC];
#pragma unroll
    for (int f = 0; f < FPL; ++f) {
        dwi[f] = lane_sum<T::LPR, 64>(dwi[f]);
        dwj[f] = lane_sum<T::LPR, 64>(dwj[f]);
    }
    if (lane < T::LPR) {
#pragma unroll
        for (int f = 0; f < FPL; ++f) {
            red[wave][0][q * FPL + f] = dwi[f];
            red[wave][1][q * FPL + f] = dwj[f];
        }
    }
    __syncthreads();
    for (int k = threadIdx.x; k < 2 * EC; k += kBlockThreads) {
        const int half = k / EC, f = k - half * EC;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) sum += red[w][half][f];
        A.dw_partials[(int64_t)blockIdx.x * (2 * A.E) + (int64_t)half * A.E + (int64_t)head * EC + f] = oa * sum;
    }
}

}  // namespace ncn
