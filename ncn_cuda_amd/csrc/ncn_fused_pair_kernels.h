// Multi-stage (LDS-resident) passes for groups of TWO rows under the stride permutation.
//
// Slot 0 of group g is row 0 of block g in every stage (torch_ref/ncn_pytorch.py:38-40: the permutation moves slot o by
// o * stride blocks), so with two rows per group half of a window never changes hands between the stages of a pass:
// the slot-0 rows stay in the registers of the lanes that own their groups from the window's load to its store, and
// only the slot-1 rows, whose partner changes with the stride, go through LDS.  Against the general kernels of
// ncn_fused_kernels.h (which these replace for n_cache = 2; same planner, same arguments) that halves the LDS
// traffic and the row addressing of a stage, and the LDS footprint of a window: a workgroup holds windows twice as
// large in the same LDS, so the halo of a pass is a smaller share of it and a stage range needs fewer passes.
// Tile shape: 2 rows x 4 features per lane (the one-stage table's), so a group is Ec/4 lanes and the pivot row is
// always in the lane itself.
#pragma once
#include "ncn_fused_kernels.h"

namespace ncn {

// One window per workgroup: the forward is launched with as many workgroups as windows, the backward too whenever
// the dW scratch has a partial row for each (LOOP = false).  Workgroups that come and go on their own fall out of step
// with the other workgroup of their CU, so that the loads and stores of one run under the stages of the other, and
// straight-line code needs no registers for what a loop over windows would carry around it (backward: 128 registers and
// no spill, against 26 spilled registers inside the loop; forward 84 against 125).  The LOOP build of the backward, for
// problems with more windows than partial rows, walks its windows with the next one's slot-1 rows requested before the
// current one is written out.
// Measured on the 13-stage configuration (x[128, 8192, 128], A/B on one box; the general kernels 6.02 ms per step):
// windows as there (64 KB of rows counting both halves) 5.70 - 5.85; windows of 128 KB (the LDS holds half: two
// workgroups per CU as in the general kernels) forward 5.51, backward too 5.33; a 256 KB forward window (one workgroup
// per CU) 6.55; forcing 6 or 8 waves per SIMD where the code does not fit (spills) 6.2 - 11.6; all of these with grids
// of 4096 workgroups that loop over 4.5 windows each.  One window per workgroup with the loop still compiled in 4.92;
// without it 4.68.
#ifndef NCN_PAIR_FWD_WAVES
#define NCN_PAIR_FWD_WAVES 4     // waves per SIMD the forward is compiled for (register budget)
#endif
#ifndef NCN_PAIR_BWD_WAVES
#define NCN_PAIR_BWD_WAVES 4
#endif
constexpr int kPairWavesBwd = kFusedWavesBwd;   // waves per workgroup of the backward

// wave tiles per wave and stage at the largest window (forward: 128 KB of rows = 256 groups at Ec = 32 over 8 waves
// of 8 groups = 4; backward: 128 groups = 2)
constexpr int kPairTilesFwd = (int)(kPairStateBytesFwd / (2 * 2 * 4 * 4 * 64 * kFusedWavesFwd));
constexpr int kPairTilesBwd = (int)((kPairStateBytesBwd + 4 * 2 * 4 * 4 * 64 * kPairWavesBwd - 1) / (4 * 2 * 4 * 4 * 64 * kPairWavesBwd));
static_assert(kPairTilesFwd >= 1 && kPairTilesBwd >= 1, "a window holds at least one wave tile per wave");

// Chunk offsets of the slot-1 rows of a window (row 1 of window sub-block qi is local row 2 qi + 1), for the
// cooperative loads: 4 features per thread and trip.
template <int EC, int NW, int K>
__device__ __forceinline__ void pair_slot1_offsets(const FusedArgs& A, const FusedItem& it, uint32_t window,
                                                   int64_t (&off)[K]) {
    constexpr uint32_t CPR = EC / 4;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = min(threadIdx.x + k * 64 * NW, window * CPR - 1u);   // past the end: re-read, ignored later
        const uint32_t qi = c / CPR, c4 = c - qi * CPR;
        off[k] = fused_row_offset<2, false>(A, it, 2u * qi + 1u) + c4 * 4;
    }
}

// Offsets of this lane's fragments of the slot-0 rows of its groups: tile k of wave w is groups (w + k NW) GPW ..
template <int EC, int NW, int KT>
__device__ __forceinline__ void pair_slot0_offsets(const FusedArgs& A, const FusedItem& it, uint32_t window, int wave,
                                                   int gw, int fl, int64_t (&off)[KT]) {
    constexpr uint32_t GPW = 64 / (EC / 4);
#pragma unroll
    for (int k = 0; k < KT; ++k) {
        const uint32_t q = min((uint32_t)(wave + k * NW) * GPW + gw, window - 1u);
        off[k] = fused_row_offset<2, false>(A, it, 2u * q) + fl * 4;
    }
}

template <int EC, int NW, int K>
__device__ __forceinline__ void pair_commit_slot1(const uint4 (&raw)[K], int dtype, float* dst, uint32_t window,
                                                  float scale) {
    constexpr uint32_t CPR = EC / 4;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = threadIdx.x + k * 64 * NW;
        if (c < window * CPR) {
            float v[4];
            fused_raw_to_float(raw[k], dtype, v);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] *= scale;
            lds_store_frag<4>(dst + c * 4, v);   // row qi, chunk c4: c * 4 == qi * EC + c4 * 4
        }
    }
}

// window position of the sub-block that holds slot 1 of the group whose slot 0 is sub-block q
__device__ __forceinline__ uint32_t pair_partner(const FusedArgs& A, uint32_t q, uint32_t ss) {
    uint32_t qi = q + ss;
    if (A.closed) qi = (q & ~(A.ring - 1u)) | (qi & (A.ring - 1u));   // wrap inside the group's own ring
    return qi;
}

// forward, and with INVERSE the same passes undone (stages last to first)
template <int EC, bool TANH_ONLY, bool INVERSE = false, bool LENGTHS = false>
__global__ void __launch_bounds__(64 * kFusedWavesFwd, NCN_PAIR_FWD_WAVES) pair_forward_kernel(const FusedArgs A) {
    constexpr int NC = 2, R = 2, F = 4, NW = kFusedWavesFwd, KT = kPairTilesFwd;
    using T = Tile<NC, EC, R, F>;
    static_assert(T::LR == 1, "both rows of a group in one lane");
    constexpr uint32_t CPR = EC / 4;
    extern __shared__ float4 fused_lds4[];
    float* lds = reinterpret_cast<float*>(fused_lds4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fl = lane % T::LF, gw = lane / T::LF;
    const uint32_t window = A.window;
    float* xs1 = lds;                               // slot-1 rows, [sub-block][EC]
    float* as1 = xs1 + window * EC;
    float* w_lds = as1 + window * EC;               // [kFusedMaxStages][2][EC]
    fused_load_weights<EC, NW>(A, blockIdx.x % A.n_head, w_lds);
    const float a_in = INVERSE ? A.tab.b_scale : A.tab.a_scale, a_out = INVERSE ? A.tab.inv_b_scale : A.tab.inv_a_scale;

    constexpr int K1 = (int)((kPairStateBytesFwd / 4 / sizeof(float4) + 64 * NW - 1) / (64 * NW));   // half the rows
    uint4 r1x[K1], r1a[K1], r0x[KT], r0a[KT];
    auto fetch = [&](uint32_t item) {
        const FusedItem nx = fused_item<NC, EC, false>(A, item);
        int64_t off1[K1], off0[KT];
        pair_slot1_offsets<EC, NW, K1>(A, nx, window, off1);
        pair_slot0_offsets<EC, NW, KT>(A, nx, window, wave, gw, fl, off0);
        fused_fetch_rows<K1>(A.in0, A.in_dtype, off1, r1x);
        fused_fetch_rows<K1>(A.in1, A.in_dtype, off1, r1a);
        fused_fetch_rows<KT>(A.in0, A.in_dtype, off0, r0x);
        fused_fetch_rows<KT>(A.in1, A.in_dtype, off0, r0a);
    };
    const uint32_t item = blockIdx.x;   // the launch has a workgroup for every window
    if (item < A.total_items) {
        const FusedItem it = fused_item<NC, EC, false>(A, item);
        const int32_t len = LENGTHS ? max(0, min(A.ctx_len[it.batch], (int32_t)A.N)) : 0;
        float x0[KT][F], a0[KT][F];   // slot-0 rows of this lane's groups, scaled form
        fetch(item);
        pair_commit_slot1<EC, NW, K1>(r1x, A.in_dtype, xs1, window, A.tab.kappa);
        pair_commit_slot1<EC, NW, K1>(r1a, A.in_dtype, as1, window, a_in);
#pragma unroll
        for (int k = 0; k < KT; ++k) {
            fused_raw_to_float(r0x[k], A.in_dtype, x0[k]);
            fused_raw_to_float(r0a[k], A.in_dtype, a0[k]);
#pragma unroll
            for (int f = 0; f < F; ++f) {
                x0[k][f] *= A.tab.kappa;
                a0[k][f] *= a_in;
            }
        }
        __syncthreads();
        for (int sq = 0; sq < A.n_stages; ++sq) {
            const int st = INVERSE ? A.n_stages - 1 - sq : sq;
            const uint32_t ss = A.sub_stride[st];
            const uint32_t ngroups = A.closed ? window : window - ss;
            float wi[F], wj[F];
            lds_load_frag<F>(w_lds + st * 2 * EC + fl * F, wi);
            lds_load_frag<F>(w_lds + st * 2 * EC + EC + fl * F, wj);
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                const uint32_t q = (uint32_t)(wave + k * NW) * T::GPW + gw;
                if ((uint32_t)(wave + k * NW) * T::GPW >= ngroups) continue;   // the same for the whole wave
                const bool valid = q < ngroups;
                const uint32_t row1 = pair_partner(A, valid ? q : 0u, ss) * EC + fl * F;
                float x[R][F], a[R][F];
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    x[0][f] = x0[k][f];
                    a[0][f] = a0[k][f];
                }
                lds_load_frag<F>(xs1 + row1, x[1]);
                lds_load_frag<F>(as1 + row1, a[1]);
                const int live = !LENGTHS ? NC : valid ? fused_live_rows<NC>(A, it, q, len) : 0;
                if (INVERSE) inverse_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x, a, wi, wj, A.tab, lane, nullptr, live);
                else forward_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x, a, wi, wj, A.tab, lane, nullptr, live);
                if (valid && (!LENGTHS || live > 0)) {
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        x0[k][f] = x[0][f];
                        a0[k][f] = a[0][f];
                    }
                    if (!LENGTHS || live > 1) {
                        lds_store_frag<F>(xs1 + row1, x[1]);
                        lds_store_frag<F>(as1 + row1, a[1]);
                    }
                }
            }
            __syncthreads();
        }
        // owned rows out of the scaled form: slot 1 from LDS, slot 0 from the registers
        for (uint32_t c = threadIdx.x; c < it.own_cnt * CPR; c += 64 * NW) {
            const uint32_t qi = it.own_lo + c / CPR, c4 = c % CPR;
            const int64_t off = fused_row_offset<NC, false>(A, it, 2u * qi + 1u) + c4 * 4;
            float v[4], u[4];
            lds_load_frag<4>(xs1 + qi * EC + c4 * 4, v);
            lds_load_frag<4>(as1 + qi * EC + c4 * 4, u);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] *= A.tab.inv_kappa;
                u[e] *= a_out;
            }
            store_frag<4>(A.out0, A.out_dtype, off, true, v);
            store_frag<4>(A.out1, A.out_dtype, off, true, u);
            if (A.aux0) {
                store_frag<4>(A.aux0, NCN_F32, off, true, v);
                store_frag<4>(A.aux1, NCN_F32, off, true, u);
            }
        }
#pragma unroll
        for (int k = 0; k < KT; ++k) {
            const uint32_t q = (uint32_t)(wave + k * NW) * T::GPW + gw;
            if (q < window && q - it.own_lo < it.own_cnt) {   // unsigned: own_lo <= q < own_lo + own_cnt
                const int64_t off = fused_row_offset<NC, false>(A, it, 2u * q) + fl * 4;
                float v[4], u[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = x0[k][e] * A.tab.inv_kappa;
                    u[e] = a0[k][e] * a_out;
                }
                store_frag<4>(A.out0, A.out_dtype, off, true, v);
                store_frag<4>(A.out1, A.out_dtype, off, true, u);
                if (A.aux0) {
                    store_frag<4>(A.aux0, NCN_F32, off, true, v);
                    store_frag<4>(A.aux1, NCN_F32, off, true, u);
                }
            }
        }
    }
}

template <int EC, bool TANH_ONLY, bool LENGTHS = false, bool LOOP = false>
__global__ void __launch_bounds__(64 * kPairWavesBwd, TANH_ONLY ? NCN_PAIR_BWD_WAVES : 1) pair_backward_kernel(const FusedArgs A) {
    constexpr int NC = 2, R = 2, F = 4, NW = kPairWavesBwd, KT = kPairTilesBwd;
    using T = Tile<NC, EC, R, F>;
    static_assert(T::LR == 1, "both rows of a group in one lane");
    constexpr uint32_t CPR = EC / 4;
    extern __shared__ float4 fused_lds4[];
    float* lds = reinterpret_cast<float*>(fused_lds4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fl = lane % T::LF, gw = lane / T::LF;
    const uint32_t window = A.window;
    const float om = 1.0f - A.tab.m;
    float* ys1 = lds;                                // slot-1 rows, [sub-block][EC]
    float* bs1 = ys1 + window * EC;
    float* gs1 = bs1 + window * EC;
    float* ps1 = gs1 + window * EC;                  // p = (1-m) g + h
    float* w_lds = ps1 + window * EC;                // [kFusedMaxStages][2][EC]
    float* dw_all = w_lds + kFusedMaxStages * 2 * EC;   // [wave][stage][2][EC]
    const int dw_wave_stride = A.n_stages * 2 * EC;
    float* dw_mine = dw_all + wave * dw_wave_stride;
    for (int k = lane; k < dw_wave_stride; k += 64) dw_mine[k] = 0.f;
    const int head = blockIdx.x % A.n_head;   // == head of every item of this workgroup (gridDim.x % n_head == 0)
    fused_load_weights<EC, NW>(A, head, w_lds);

    constexpr int K1 = (int)((kPairStateBytesBwd / 8 / sizeof(float4) + 64 * NW - 1) / (64 * NW));   // half the rows
    // The slot-1 rows of the next window are requested before the current one is written out and land in LDS after it
    // (raw bits in registers meanwhile); the slot-0 rows go straight into the registers that hold them, once those are
    // free, i.e. after the write-out.
    struct Raw {
        uint4 y1[K1], b1[K1], g1[K1], h1[K1];
    };
    auto fetch = [&](uint32_t item, Raw& r) {
        const FusedItem nx = fused_item<NC, EC, false>(A, item);
        int64_t off1[K1];
        pair_slot1_offsets<EC, NW, K1>(A, nx, window, off1);
        fused_fetch_rows<K1>(A.in0, A.in_dtype, off1, r.y1);
        fused_fetch_rows<K1>(A.in1, A.in_dtype, off1, r.b1);
        fused_fetch_rows<K1>(A.g0, A.g_dtype, off1, r.g1);
        fused_fetch_rows<K1>(A.g1, A.g_dtype, off1, r.h1);
    };
    float Y0[KT][F], B0[KT][F], G0[KT][F], P0[KT][F];   // slot-0 rows of this lane's groups: xs, bh, g / m^t, p / m^t
    auto commit = [&](const Raw& r) {
        pair_commit_slot1<EC, NW, K1>(r.y1, A.in_dtype, ys1, window, A.tab.kappa);
        pair_commit_slot1<EC, NW, K1>(r.b1, A.in_dtype, bs1, window, A.tab.b_scale);
        pair_commit_slot1<EC, NW, K1>(r.g1, A.g_dtype, gs1, window, 1.0f);
#pragma unroll
        for (int k = 0; k < K1; ++k) {   // p = (1-m) g + h  (h = 0 when dya is null: the fetch left zeros)
            const uint32_t c = threadIdx.x + k * 64 * NW;
            if (c < window * CPR) {
                float g[4], h[4];
                fused_raw_to_float(r.g1[k], A.g_dtype, g);
                fused_raw_to_float(r.h1[k], A.g_dtype, h);
#pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = fmaf(om, g[e], h[e]);
                lds_store_frag<4>(ps1 + c * 4, h);
            }
        }
    };
    auto load_slot0 = [&](uint32_t item) {
        const FusedItem nx = fused_item<NC, EC, false>(A, item);
        int64_t off0[KT];
        pair_slot0_offsets<EC, NW, KT>(A, nx, window, wave, gw, fl, off0);
        uint4 ry[KT], rb[KT], rg[KT], rh[KT];
        fused_fetch_rows<KT>(A.in0, A.in_dtype, off0, ry);
        fused_fetch_rows<KT>(A.in1, A.in_dtype, off0, rb);
        fused_fetch_rows<KT>(A.g0, A.g_dtype, off0, rg);
        fused_fetch_rows<KT>(A.g1, A.g_dtype, off0, rh);
#pragma unroll
        for (int k = 0; k < KT; ++k) {
            float h[4];
            fused_raw_to_float(ry[k], A.in_dtype, Y0[k]);
            fused_raw_to_float(rb[k], A.in_dtype, B0[k]);
            fused_raw_to_float(rg[k], A.g_dtype, G0[k]);
            fused_raw_to_float(rh[k], A.g_dtype, h);
#pragma unroll
            for (int f = 0; f < F; ++f) {
                Y0[k][f] *= A.tab.kappa;
                B0[k][f] *= A.tab.b_scale;
                P0[k][f] = fmaf(om, G0[k][f], h[f]);
            }
        }
    };
    if (blockIdx.x < A.total_items) {
        Raw first;
        fetch(blockIdx.x, first);
        load_slot0(blockIdx.x);
        commit(first);
    }
    __syncthreads();
    uint32_t item = blockIdx.x;
    if (item < A.total_items) do {
        const FusedItem it = fused_item<NC, EC, false>(A, item);
        const int32_t len = LENGTHS ? max(0, min(A.ctx_len[it.batch], (int32_t)A.N)) : 0;
        for (int st = A.n_stages - 1; st >= 0; --st) {
            const uint32_t ss = A.sub_stride[st];
            const uint32_t ngroups = A.closed ? window : window - ss;
            float wi[F], wj[F], dwi[F], dwj[F];
            lds_load_frag<F>(w_lds + st * 2 * EC + fl * F, wi);
            lds_load_frag<F>(w_lds + st * 2 * EC + EC + fl * F, wj);
#pragma unroll
            for (int f = 0; f < F; ++f) dwi[f] = dwj[f] = 0.f;
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                const uint32_t q = (uint32_t)(wave + k * NW) * T::GPW + gw;
                if ((uint32_t)(wave + k * NW) * T::GPW >= ngroups) continue;   // the same for the whole wave
                const bool valid = q < ngroups;
                const float own = (valid && q - it.own_lo < it.own_cnt) ? 1.0f : 0.0f;  // unsigned: lo <= q < lo+cnt
                const uint32_t row1 = pair_partner(A, valid ? q : 0u, ss) * EC + fl * F;
                float Y[R][F], B[R][F], G[R][F], P[R][F];
                lds_load_frag<F>(ys1 + row1, Y[1]);
                lds_load_frag<F>(bs1 + row1, B[1]);
                lds_load_frag<F>(gs1 + row1, G[1]);
                lds_load_frag<F>(ps1 + row1, P[1]);
                const int live = !LENGTHS ? NC : valid ? fused_live_rows<NC>(A, it, q, len) : 0;
                if (LENGTHS && live == 0 && valid) {
                    // the whole group is past the length: its gradients only take the stage's power of 1/m
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        G0[k][f] *= A.tab.inv_m_pow_n;
                        P0[k][f] *= A.tab.inv_m_pow_n;
                    }
                }
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const bool on = !LENGTHS || live > 0;
                    Y[0][f] = on ? Y0[k][f] : 0.f;
                    B[0][f] = on ? B0[k][f] : 0.f;
                    G[0][f] = on ? G0[k][f] : 0.f;
                    P[0][f] = on ? P0[k][f] : 0.f;
                }
                if (LENGTHS && live != NC) {
                    // G, P carry m^-t: the steps this group skips still count (see the general kernels)
                    const float isc = pow_steps(A.tab.im, NC - live);
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        G[0][f] *= isc;
                        P[0][f] *= isc;
                        G[1][f] *= A.tab.inv_m_pow_n;   // slot 1 is past the length whenever the group is cut
                        P[1][f] *= A.tab.inv_m_pow_n;
                    }
                    if (valid) {
                        lds_store_frag<F>(gs1 + row1, G[1]);
                        lds_store_frag<F>(ps1 + row1, P[1]);
                    }
#pragma unroll
                    for (int f = 0; f < F; ++f) Y[1][f] = B[1][f] = G[1][f] = P[1][f] = 0.f;
                }
                backward_core<NC, EC, R, F, true, TANH_ONLY, LENGTHS, true>(Y, B, G, P, wi, wj, dwi, dwj, own, A.tab,
                                                                          (A.n_stages - 1 - st) * NC, lane, nullptr, live);
                if (valid && (!LENGTHS || live > 0)) {
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        Y0[k][f] = Y[0][f];
                        B0[k][f] = B[0][f];
                        G0[k][f] = G[0][f];
                        P0[k][f] = P[0][f];
                    }
                    if (!LENGTHS || live > 1) {
                        lds_store_frag<F>(ys1 + row1, Y[1]);
                        lds_store_frag<F>(bs1 + row1, B[1]);
                        lds_store_frag<F>(gs1 + row1, G[1]);
                        lds_store_frag<F>(ps1 + row1, P[1]);
                    }
                }
            }
            // this wave's dW share of the stage (as in the general kernels: lanes of each half of the wave that hold
            // the same features, then the two halves add to the wave's slot one after the other)
#pragma unroll
            for (int f = 0; f < F; ++f) {
                dwi[f] = lane_sum<T::LF, 32, true>(dwi[f]);
                dwj[f] = lane_sum<T::LF, 32, true>(dwj[f]);
            }
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                if (lane == fl + 32 * half) {
                    float* d = dw_mine + st * (2 * EC) + fl * F;
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        d[f] += dwi[f];
                        d[EC + f] += dwj[f];
                    }
                }
            }
            __syncthreads();
        }
        auto write_out = [&]() {   // owned rows back to true values: g = G m^T, h = P m^T - (1-m) g, x = xs / kappa, xa = bh / b_scale
            for (uint32_t c = threadIdx.x; c < it.own_cnt * CPR; c += 64 * NW) {
                const uint32_t qi = it.own_lo + c / CPR, c4 = c % CPR;
                const int64_t off = fused_row_offset<NC, false>(A, it, 2u * qi + 1u) + c4 * 4;
                float g[4], h[4];
                lds_load_frag<4>(gs1 + qi * EC + c4 * 4, g);
                lds_load_frag<4>(ps1 + qi * EC + c4 * 4, h);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    g[e] *= A.scale_dn;
                    h[e] = fmaf(h[e], A.scale_dn, -om * g[e]);
                }
                store_frag<4>(A.out0, A.out_dtype, off, true, g);
                store_frag<4>(A.out1, A.out_dtype, off, true, h);
                if (A.aux0) {
                    float y[4], b[4];
                    lds_load_frag<4>(ys1 + qi * EC + c4 * 4, y);
                    lds_load_frag<4>(bs1 + qi * EC + c4 * 4, b);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        y[e] *= A.tab.inv_kappa;
                        b[e] *= A.tab.inv_b_scale;
                    }
                    store_frag<4>(A.aux0, NCN_F32, off, true, y);
                    store_frag<4>(A.aux1, NCN_F32, off, true, b);
                }
            }
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                const uint32_t q = (uint32_t)(wave + k * NW) * T::GPW + gw;
                if (q < window && q - it.own_lo < it.own_cnt) {
                    const int64_t off = fused_row_offset<NC, false>(A, it, 2u * q) + fl * 4;
                    float g[4], h[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        g[e] = G0[k][e] * A.scale_dn;
                        h[e] = fmaf(P0[k][e], A.scale_dn, -om * g[e]);
                    }
                    store_frag<4>(A.out0, A.out_dtype, off, true, g);
                    store_frag<4>(A.out1, A.out_dtype, off, true, h);
                    if (A.aux0) {
                        float y[4], b[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            y[e] = Y0[k][e] * A.tab.inv_kappa;
                            b[e] = B0[k][e] * A.tab.inv_b_scale;
                        }
                        store_frag<4>(A.aux0, NCN_F32, off, true, y);
                        store_frag<4>(A.aux1, NCN_F32, off, true, b);
                    }
                }
            }
        };
        if (LOOP && item + gridDim.x < A.total_items) {   // the same for the whole workgroup
            Raw next;
            fetch(item + gridDim.x, next);
            write_out();
            load_slot0(item + gridDim.x);
            __syncthreads();   // every thread has read what it writes out: the window may be overwritten
            commit(next);
        } else {
            write_out();
        }
        __syncthreads();
    } while (LOOP && (item += gridDim.x) < A.total_items);
    // one partial row per workgroup and stage; workgroup b owns slot (b / n_head, head b % n_head)
    float* prow = A.dw_partials + (int64_t)(blockIdx.x / A.n_head) * A.n_stages * (2 * A.E);
    for (int k = threadIdx.x; k < A.n_stages * 2 * EC; k += 64 * NW) {
        const int st = k / (2 * EC), rem = k - st * 2 * EC, half = rem / EC, f = rem - half * EC;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += dw_all[w * dw_wave_stride + st * 2 * EC + rem];
        prow[(int64_t)st * (2 * A.E) + (int64_t)half * A.E + (int64_t)head * EC + f] = sum;
    }
}

}  // namespace ncn
