// Multi-stage (LDS-resident) passes for groups of TWO rows under the stride permutation.
//
// Slot 0 of group g is row 0 of block g in every stage (torch_ref/ncn_pytorch.py:38-40: the permutation moves slot o by
// o * stride blocks), so with two rows per group half of a window never changes hands between the stages of a pass:
// the slot-0 rows stay in the registers of the lanes that own their groups from the window's load to its store, and
// only the slot-1 rows, whose partner changes with the stride, go through LDS.  Against the general kernels of
// ncn_fused_kernels.h (which these replace for n_cache = 2; same planner, same arguments) that halves the LDS
// traffic and the row addressing of a stage, and the LDS footprint of a window: a workgroup holds windows twice as
// large in the same LDS, so the halo of a pass is a smaller share of it and a stage range needs fewer passes.
// Both rows of a group are in one lane, so the pivot row is always in the lane itself.
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

// Tile shape: 2 rows x F features per lane, F = 8 where the head is that wide (4 lanes per row at 32 features: the
// row sums of a step cross two DPP levels instead of three, and the per-row, per-step and per-tile bookkeeping is
// spread over twice the elements).  A lane's F features are F/4 chunks of 4: chunk h of feature lane fl is chunk
// fl + h * LF of the row, so the lanes of a row cover LF * 16 contiguous bytes with every 16-byte access.
template <int EC>
struct PairShape {
    static constexpr int F = EC >= 8 ? 8 : 4;
    static constexpr int H = F / 4;          // 16-byte chunks per lane and row
    static constexpr int LF = EC / F;        // lanes per row == lanes per group
    static constexpr int GPW = 64 / LF;      // groups per wave tile
};

// wave tiles per wave and stage at the largest window
template <int EC>
constexpr int pair_tiles(bool backward) {
    const size_t per_tile = (size_t)(backward ? 4 : 2) * 2 * PairShape<EC>::F * 4 * 64 * (backward ? kPairWavesBwd : kFusedWavesFwd);
    const size_t state = backward ? kPairStateBytesBwd : kPairStateBytesFwd;
    return (int)((state + per_tile - 1) / per_tile);
}

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

// Offsets of this lane's chunks of the slot-0 rows of its groups: tile k of wave w is groups (w + k NW) GPW ..
template <int EC, int NW, int KT>
__device__ __forceinline__ void pair_slot0_offsets(const FusedArgs& A, const FusedItem& it, uint32_t window, int wave,
                                                   int gw, int fl, int64_t (&off)[KT * PairShape<EC>::H]) {
    using S = PairShape<EC>;
#pragma unroll
    for (int k = 0; k < KT; ++k) {
        const uint32_t q = min((uint32_t)(wave + k * NW) * S::GPW + gw, window - 1u);
        const int64_t row = fused_row_offset<2, false>(A, it, 2u * q);
#pragma unroll
        for (int h = 0; h < S::H; ++h) off[k * S::H + h] = row + (fl + h * S::LF) * 4;
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
    return A.closed ? ring_wrap(A, q, ss) : q + ss;   // closed: inside the group's own ring
}

// a lane's F features of an LDS row (or of a weight vector): its H chunks of 4
template <int EC>
__device__ __forceinline__ void pair_lds_load(const float* row, int fl, float (&v)[PairShape<EC>::F]) {
    using S = PairShape<EC>;
#pragma unroll
    for (int h = 0; h < S::H; ++h) {
        const float4 t = *reinterpret_cast<const float4*>(row + (fl + h * S::LF) * 4);
        v[4 * h] = t.x; v[4 * h + 1] = t.y; v[4 * h + 2] = t.z; v[4 * h + 3] = t.w;
    }
}
template <int EC>
__device__ __forceinline__ void pair_lds_store(float* row, int fl, const float (&v)[PairShape<EC>::F]) {
    using S = PairShape<EC>;
#pragma unroll
    for (int h = 0; h < S::H; ++h)
        *reinterpret_cast<float4*>(row + (fl + h * S::LF) * 4) = make_float4(v[4 * h], v[4 * h + 1], v[4 * h + 2], v[4 * h + 3]);
}

// forward, and with INVERSE the same passes undone (stages last to first)
template <int EC, bool TANH_ONLY, bool INVERSE = false, bool LENGTHS = false, bool HEADWISE = false>
__global__ void __launch_bounds__(64 * kFusedWavesFwd, NCN_PAIR_FWD_WAVES) pair_forward_kernel(const FusedArgs A) {
    using S = PairShape<EC>;
    constexpr int NC = 2, R = 2, F = S::F, H = S::H, NW = kFusedWavesFwd, KT = pair_tiles<EC>(false);
    using T = Tile<NC, EC, R, F>;
    static_assert(T::LR == 1, "both rows of a group in one lane");
    constexpr uint32_t CPR = EC / 4;
    extern __shared__ float4 fused_lds4[];
    float* lds = reinterpret_cast<float*>(fused_lds4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fl = lane % T::LF, gw = lane / T::LF;
    const uint32_t window = A.window;
    // the arrays lie a fixed distance apart (the largest window's), so that one address register serves them all
    constexpr uint32_t ARR = kPairStateBytesFwd / 4 / sizeof(float);
    float* xs1 = lds;                               // slot-1 rows, [sub-block][EC]
    float* as1 = xs1 + ARR;
    float* w_lds = as1 + ARR;                       // [kFusedMaxStages][2][EC]
    fused_load_weights<EC, NW>(A, blockIdx.x % A.n_head, w_lds);
    const float a_in = INVERSE ? A.tab.b_scale : A.tab.a_scale, a_out = INVERSE ? A.tab.inv_b_scale : A.tab.inv_a_scale;

    constexpr int K1 = (int)((kPairStateBytesFwd / 4 / sizeof(float4) + 64 * NW - 1) / (64 * NW));   // half the rows
    const uint32_t item = blockIdx.x;   // the launch has a workgroup for every window
    if (item < A.total_items) {
        const FusedItem it = fused_item<NC, EC, false>(A, item);
        const int32_t len = LENGTHS ? max(0, min(A.ctx_len[it.batch], (int32_t)A.N)) : 0;
        // rows of this lane's groups in the scaled form: [k][0] the slot-0 row, which stays here from the window's
        // load to its store; [k][1] the slot-1 row, which every stage takes from LDS and puts back
        float x[KT][R][F], a[KT][R][F];
        {
            uint4 r1x[K1], r1a[K1], r0x[KT * H], r0a[KT * H];
            int64_t off1[K1], off0[KT * H];
            pair_slot1_offsets<EC, NW, K1>(A, it, window, off1);
            pair_slot0_offsets<EC, NW, KT>(A, it, window, wave, gw, fl, off0);
            fused_fetch_rows<K1>(A.in0, A.in_dtype, off1, r1x);
            fused_fetch_rows<K1>(A.in1, A.in_dtype, off1, r1a);
            fused_fetch_rows<KT * H>(A.in0, A.in_dtype, off0, r0x);
            fused_fetch_rows<KT * H>(A.in1, A.in_dtype, off0, r0a);
            pair_commit_slot1<EC, NW, K1>(r1x, A.in_dtype, xs1, window, A.tab.kappa);
            pair_commit_slot1<EC, NW, K1>(r1a, A.in_dtype, as1, window, a_in);
#pragma unroll
            for (int k = 0; k < KT; ++k)
#pragma unroll
                for (int h = 0; h < H; ++h) {
                    float vx[4], va[4];
                    fused_raw_to_float(r0x[k * H + h], A.in_dtype, vx);
                    fused_raw_to_float(r0a[k * H + h], A.in_dtype, va);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        x[k][0][4 * h + e] = vx[e] * A.tab.kappa;
                        a[k][0][4 * h + e] = va[e] * a_in;
                    }
                }
        }
        __syncthreads();
        for (int sq = 0; sq < A.n_stages; ++sq) {
            const int st = INVERSE ? A.n_stages - 1 - sq : sq;
            const uint32_t ss = A.sub_stride[st];
            const uint32_t ngroups = A.closed ? window : window - ss;
            float wi[F], wj[F];
            pair_lds_load<EC>(w_lds + st * 2 * EC, fl, wi);
            pair_lds_load<EC>(w_lds + st * 2 * EC + EC, fl, wj);
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                const uint32_t q = (uint32_t)(wave + k * NW) * T::GPW + gw;
                // Lanes whose group does not exist in this stage (past the last group that lies inside the window)
                // sit the tile out: every cross-lane sum of a step stays inside one group, so no lane a live group
                // needs is off, and the rows of the lanes that are off keep their values.
                if (q < ngroups) {
                    const uint32_t row1 = pair_partner(A, q, ss) * EC;
                    pair_lds_load<EC>(xs1 + row1, fl, x[k][1]);
                    pair_lds_load<EC>(as1 + row1, fl, a[k][1]);
                    const int live = !LENGTHS ? NC : fused_live_rows<NC>(A, it, q, len);
                    if constexpr (HEADWISE) {
                        if (INVERSE) headwise_inverse_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x[k], a[k], wi, wj, A.tab, lane, nullptr, live);
                        else headwise_forward_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x[k], a[k], wi, wj, A.tab, lane, nullptr, live);
                    } else {
                        if (INVERSE) inverse_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x[k], a[k], wi, wj, A.tab, lane, nullptr, live);
                        else forward_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x[k], a[k], wi, wj, A.tab, lane, nullptr, live);
                    }
                    if (!LENGTHS || live > 1) {
                        pair_lds_store<EC>(xs1 + row1, fl, x[k][1]);
                        pair_lds_store<EC>(as1 + row1, fl, a[k][1]);
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
                const int64_t row = fused_row_offset<NC, false>(A, it, 2u * q);
#pragma unroll
                for (int h = 0; h < H; ++h) {
                    const int64_t off = row + (fl + h * T::LF) * 4;
                    float v[4], u[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = x[k][0][4 * h + e] * A.tab.inv_kappa;
                        u[e] = a[k][0][4 * h + e] * a_out;
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
}

// Sums each of the NV values v[.] over the lanes of the wave that hold the same features (one lane of every group of
// the wave tile) and scatters the sums: afterwards v[0 .. pair_scatter_left) of a lane are complete, and they are the
// values number `first` and up of the original list, where `first` (returned) depends on the lane.  Every level
// halves the list a lane carries on: the lanes on one side of the level's lane bit keep the lower half, the others the
// upper half, and each adds what the other side sends it.  Across half-waves and across rows of 16 lanes that is one
// swap of two registers' halves (v_permlane32_swap / v_permlane16_swap) and one add per two values; inside a row two
// DPP moves whose write masks pick the side and one add.  (Summing every value in every lane costs one instruction
// per value and level: 3 levels x 16 values against 33 instructions here at 4 lanes per group.)
template <int LF>
constexpr int pair_scatter_levels() { return LF <= 4 ? 4 : LF == 8 ? 3 : 2; }   // lane bits 5, 4 and, where they are group bits, 3 and 2
template <int LF, int NV>
constexpr int pair_scatter_left() { return NV >> pair_scatter_levels<LF>(); }

template <int LF, int NV>
__device__ __forceinline__ int pair_scatter_sum(float (&v)[NV], int lane) {
    static_assert(LF == 1 || LF == 2 || LF == 4 || LF == 8 || LF == 16, "lanes per group");
    static_assert(NV == 16, "two rows of 8 weights");
    // lane bit 5: lower half-wave keeps v[0..8), upper v[8..16)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[i]), __float_as_uint(v[i + 8]), false, false);
        v[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    // lane bit 4: even rows keep v[0..4), odd rows v[4..8)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v[i]), __float_as_uint(v[i + 4]), false, false);
        v[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    int first = ((lane >> 5) & 1) * 8 + ((lane >> 4) & 1) * 4;
    if constexpr (LF <= 8) {
        // lane bit 3: banks 0,1 of a row keep v[0..2), banks 2,3 keep v[2..4); row_ror:8 reads lane (l + 8) mod 16
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int lo = __float_as_int(v[i]), hi = __float_as_int(v[i + 2]);
            const int t = __builtin_amdgcn_update_dpp(hi, lo, 0x128, 0xF, 0x3, false);   // banks 0,1: partner's lo; 2,3: own hi
            const int u = __builtin_amdgcn_update_dpp(lo, hi, 0x128, 0xF, 0xC, false);   // banks 2,3: partner's hi; 0,1: own lo
            v[i] = __int_as_float(t) + __int_as_float(u);
        }
        first += ((lane >> 3) & 1) * 2;
    }
    if constexpr (LF <= 4) {
        // lane bit 2: banks 0,2 keep v[0], banks 1,3 keep v[1]; row_shl:4 reads lane l + 4, row_shr:4 lane l - 4
        const int lo = __float_as_int(v[0]), hi = __float_as_int(v[1]);
        const int t = __builtin_amdgcn_update_dpp(hi, lo, 0x104, 0xF, 0x5, false);   // banks 0,2: partner's lo; 1,3: own hi
        const int u = __builtin_amdgcn_update_dpp(lo, hi, 0x114, 0xF, 0xA, false);   // banks 1,3: partner's hi; 0,2: own lo
        v[0] = __int_as_float(t) + __int_as_float(u);
        first += (lane >> 2) & 1;
    }
    // lanes of one group that still hold shares of the same value (heads narrower than 32 features): plain sums
    if constexpr (LF <= 2) v[0] += lane_xor<2>(v[0]);
    if constexpr (LF == 1) v[0] += lane_xor<1>(v[0]);
    return first;
}

template <int EC, bool TANH_ONLY, bool LENGTHS = false, bool LOOP = false, bool HEADWISE = false>
__global__ void __launch_bounds__(64 * kPairWavesBwd, TANH_ONLY ? NCN_PAIR_BWD_WAVES : 1) pair_backward_kernel(const FusedArgs A) {
    using S = PairShape<EC>;
    constexpr int NC = 2, R = 2, F = S::F, H = S::H, NW = kPairWavesBwd, KT = pair_tiles<EC>(true);
    using T = Tile<NC, EC, R, F>;
    static_assert(T::LR == 1, "both rows of a group in one lane");
    static_assert(F == 8, "the dW sums are written for 8 features per lane");
    constexpr uint32_t CPR = EC / 4;
    extern __shared__ float4 fused_lds4[];
    float* lds = reinterpret_cast<float*>(fused_lds4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fl = lane % T::LF, gw = lane / T::LF;
    const uint32_t window = A.window;
    const float om = 1.0f - A.tab.m;
    // the arrays lie a fixed distance apart (the largest window's), so that one address register serves them all
    constexpr uint32_t ARR = kPairStateBytesBwd / 8 / sizeof(float);
    float* ys1 = lds;                                // slot-1 rows, [sub-block][EC]
    float* bs1 = ys1 + ARR;
    float* gs1 = bs1 + ARR;
    float* ps1 = gs1 + ARR;                          // p = (1-m) g + h
    float* w_lds = ps1 + ARR;                        // [kFusedMaxStages][2][EC]
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
    // rows of this lane's groups: [k][0] the slot-0 row, which stays here from the window's load to its store;
    // [k][1] the slot-1 row, which every stage takes from LDS and puts back.  xs, bh, g / m^t, p / m^t.
    float Y[KT][R][F], B[KT][R][F], G[KT][R][F], P[KT][R][F];
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
        int64_t off0[KT * H];
        pair_slot0_offsets<EC, NW, KT>(A, nx, window, wave, gw, fl, off0);
        uint4 ry[KT * H], rb[KT * H], rg[KT * H], rh[KT * H];
        fused_fetch_rows<KT * H>(A.in0, A.in_dtype, off0, ry);
        fused_fetch_rows<KT * H>(A.in1, A.in_dtype, off0, rb);
        fused_fetch_rows<KT * H>(A.g0, A.g_dtype, off0, rg);
        fused_fetch_rows<KT * H>(A.g1, A.g_dtype, off0, rh);
#pragma unroll
        for (int k = 0; k < KT; ++k)
#pragma unroll
            for (int c = 0; c < H; ++c) {
                float y[4], b[4], g[4], h[4];
                fused_raw_to_float(ry[k * H + c], A.in_dtype, y);
                fused_raw_to_float(rb[k * H + c], A.in_dtype, b);
                fused_raw_to_float(rg[k * H + c], A.g_dtype, g);
                fused_raw_to_float(rh[k * H + c], A.g_dtype, h);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    Y[k][0][4 * c + e] = y[e] * A.tab.kappa;
                    B[k][0][4 * c + e] = b[e] * A.tab.b_scale;
                    G[k][0][4 * c + e] = g[e];
                    P[k][0][4 * c + e] = fmaf(om, g[e], h[e]);
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
            float wi[F], wj[F], dw[2 * F];   // dw: this lane's share of dWi (first F) and dWj of the stage
            pair_lds_load<EC>(w_lds + st * 2 * EC, fl, wi);
            pair_lds_load<EC>(w_lds + st * 2 * EC + EC, fl, wj);
#pragma unroll
            for (int f = 0; f < 2 * F; ++f) dw[f] = 0.f;
            float (&dwi)[F] = *reinterpret_cast<float (*)[F]>(&dw[0]);
            float (&dwj)[F] = *reinterpret_cast<float (*)[F]>(&dw[F]);
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                const uint32_t q = (uint32_t)(wave + k * NW) * T::GPW + gw;
                // Lanes whose group does not exist in this stage sit the tile out (every cross-lane sum of a step
                // stays inside one group); their rows keep their values.
                if (q < ngroups) {
                    const float own = (q - it.own_lo < it.own_cnt) ? 1.0f : 0.0f;  // unsigned: lo <= q < lo + cnt
                    const uint32_t row1 = pair_partner(A, q, ss) * EC;
                    pair_lds_load<EC>(ys1 + row1, fl, Y[k][1]);
                    pair_lds_load<EC>(bs1 + row1, fl, B[k][1]);
                    pair_lds_load<EC>(gs1 + row1, fl, G[k][1]);
                    pair_lds_load<EC>(ps1 + row1, fl, P[k][1]);
                    const int live = !LENGTHS ? NC : fused_live_rows<NC>(A, it, q, len);
                    if (LENGTHS && live != NC) {
                        // G, P carry m^-t: the steps this group skips still count.  Slot 1 is past the length whenever
                        // the group is cut: it takes the power of 1/m of the whole stage, goes back to LDS and leaves
                        // the sums of the group (zeros in the registers).  Slot 0 takes the factor of the skipped
                        // steps here and that of its own step, if it is live, in the step code.
                        const float isc = live == 0 ? A.tab.inv_m_pow_n : pow_steps(A.tab.im, NC - live);
#pragma unroll
                        for (int f = 0; f < F; ++f) {
                            G[k][0][f] *= isc;
                            P[k][0][f] *= isc;
                            G[k][1][f] *= A.tab.inv_m_pow_n;
                            P[k][1][f] *= A.tab.inv_m_pow_n;
                        }
                        pair_lds_store<EC>(gs1 + row1, fl, G[k][1]);
                        pair_lds_store<EC>(ps1 + row1, fl, P[k][1]);
#pragma unroll
                        for (int f = 0; f < F; ++f) Y[k][1][f] = B[k][1][f] = G[k][1][f] = P[k][1][f] = 0.f;
                    }
                    if constexpr (HEADWISE)
                        headwise_backward_core<NC, EC, R, F, true, TANH_ONLY, LENGTHS, true, false>(
                            Y[k], B[k], G[k], P[k], wi, wj, dwi, dwj, own, A.tab, (A.n_stages - 1 - st) * NC, lane, nullptr, live);
                    else
                        backward_core<NC, EC, R, F, true, TANH_ONLY, LENGTHS, true, false>(
                            Y[k], B[k], G[k], P[k], wi, wj, dwi, dwj, own, A.tab, (A.n_stages - 1 - st) * NC, lane, nullptr, live);
                    if (!LENGTHS || live > 1) {
                        pair_lds_store<EC>(ys1 + row1, fl, Y[k][1]);
                        pair_lds_store<EC>(bs1 + row1, fl, B[k][1]);
                        pair_lds_store<EC>(gs1 + row1, fl, G[k][1]);
                        pair_lds_store<EC>(ps1 + row1, fl, P[k][1]);
                    }
                }
            }
            // this wave's dW share of the stage into its own LDS slot: every lane ends up with one or two complete
            // sums (always the same ones: the order of the additions is fixed)
            {
                const int first = pair_scatter_sum<T::LF, 2 * F>(dw, lane);
                constexpr int LEFT = pair_scatter_left<T::LF, 2 * F>();
                const int half = first / F, f0 = first % F;           // dWi or dWj; feature register f0 of the lane
                float* d = dw_mine + st * (2 * EC) + half * EC + (fl + (f0 / 4) * T::LF) * 4 + (f0 % 4);
                if (T::LF >= 4 || (lane & (T::LF == 2 ? 2 : 3)) == 0) {   // narrow heads: one lane per value writes
#pragma unroll
                    for (int i = 0; i < LEFT; ++i) d[i] += dw[i];
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
                    const int64_t row = fused_row_offset<NC, false>(A, it, 2u * q);
#pragma unroll
                    for (int c = 0; c < H; ++c) {
                        const int64_t off = row + (fl + c * T::LF) * 4;
                        float g[4], h[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            g[e] = G[k][0][4 * c + e] * A.scale_dn;
                            h[e] = fmaf(P[k][0][4 * c + e], A.scale_dn, -om * g[e]);
                        }
                        store_frag<4>(A.out0, A.out_dtype, off, true, g);
                        store_frag<4>(A.out1, A.out_dtype, off, true, h);
                        if (A.aux0) {
                            float y[4], b[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                y[e] = Y[k][0][4 * c + e] * A.tab.inv_kappa;
                                b[e] = B[k][0][4 * c + e] * A.tab.inv_b_scale;
                            }
                            store_frag<4>(A.aux0, NCN_F32, off, true, y);
                            store_frag<4>(A.aux1, NCN_F32, off, true, b);
                        }
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
