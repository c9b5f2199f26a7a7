// Heads of one feature (E == n_head: every feature is a head of its own, the recurrence on rows of scalars).
//
// A head's "dot products" are single products, so nothing is summed across the features of a row.  The register
// tiles of ncn_stage_kernels.h are kept, with a different meaning of the EC features that the LF lanes of a row hold:
// EC adjacent heads instead of one head of EC features.  The host hands these kernels E / EC "heads" of width EC
// (StageArgs.n_head, head_dim; EC = 32, 16, 8 or 4, the largest that divides E), so that tiles, offsets, weights, grids
// and the dW partial rows are laid out as for heads of EC features (a wave reads up to 128 contiguous bytes of a row),
// and the step code differs from forward_core / inverse_core / backward_core only in that the row sums c_i, rh_i are
// per-feature values c_if, rh_if that never cross lanes:
//
//   s_if = x_if Wi_f + x_jf Wj_f      T_if = alpha x_if + (1-alpha) s_if x_jf      (torch_ref/ncn_pytorch.py:74-94, Ec = 1)
//
// Per step the only traffic across lanes is the pivot row's broadcast and, in the backward, the sum of its gradient
// over the row lanes of the group.
#pragma once
#include "ncn_stage_kernels.h"

namespace ncn {

// The three functions take the template and call arguments of forward_core, inverse_core and backward_core, so that a
// kernel picks one or the other by name (ROWS only reaches the sum over a group's row lanes; KU_W has nothing to act
// on here).
template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void headwise_forward_core(float (&x)[R][F], float (&a)[R][F], const float (&wi)[F],
                                                      const float (&wj)[F], const StepTable& S, int lane, float4* slots,
                                                      int live = NC) {
    using T = Tile<NC, EC, R, F>;
#pragma unroll 1
    for (int jo = 0; jo < T::LR; ++jo) {
#pragma unroll
        for (int jr = 0; jr < R; ++jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;  // the lanes of a group agree: no lane it needs is off
            float xj[F], cj[F];
            row_lane_broadcast<T::LF, T::LR, F>(x[jr], xj, jo, lane, slots);
#pragma unroll
            for (int f = 0; f < F; ++f) cj[f] = xj[f] * wj[f];
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float c = fmaf(x[rr][f], wi[f], cj[f]);
                    const float z = fmaf(c, xj[f], x[rr][f]);
                    if constexpr (TANH_ONLY) {
                        const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
                        a[rr][f] = fmaf(S.m2k2, r, fmaf(S.m, a[rr][f], S.k2));
                    } else {
                        float Fv, w;
                        act_Fw(z, S.activation, Fv, w);
                        a[rr][f] = fmaf(S.k2, Fv, S.m * a[rr][f]);
                    }
                    x[rr][f] = fmaf(S.m, x[rr][f], a[rr][f]);
                }
            }
        }
    }
}

template <int NC, int EC, int R, int F, bool TANH_ONLY, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void headwise_inverse_core(float (&y)[R][F], float (&b)[R][F], const float (&wi)[F],
                                                      const float (&wj)[F], const StepTable& S, int lane, float4* slots,
                                                      int live = NC) {
    using T = Tile<NC, EC, R, F>;
#pragma unroll 1
    for (int jo = T::LR - 1; jo >= 0; --jo) {
#pragma unroll
        for (int jr = R - 1; jr >= 0; --jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int f = 0; f < F; ++f) y[rr][f] = fmaf(S.im, y[rr][f], -b[rr][f]);
            float xj[F], cj[F];
            row_lane_broadcast<T::LF, T::LR, F>(y[jr], xj, jo, lane, slots);
#pragma unroll
            for (int f = 0; f < F; ++f) cj[f] = xj[f] * wj[f];
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float c = fmaf(y[rr][f], wi[f], cj[f]);
                    const float z = fmaf(c, xj[f], y[rr][f]);
                    if constexpr (TANH_ONLY) {
                        const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
                        b[rr][f] = fmaf(S.bk1, r, fmaf(S.im, b[rr][f], S.bk0));
                    } else {
                        float Fv, w;
                        act_Fw(z, S.activation, Fv, w);
                        b[rr][f] = fmaf(S.bk0, Fv, S.im * b[rr][f]);
                    }
                }
            }
        }
    }
}

// The reversible backward of backward_core on the same scaled state (Y = xs, B = bh, G = g / m^t, P = p / m^t), with
//   U_if = P_if F'/4,   rh_if = U_if xs_jf,   G_if += ku (U_if + rh_if Wi'_f),   dWi_f += krho[t] rh_if xs_if,
//   pivot row:  G_jf += ku sum_i (rh_if Wj'_f + c_if U_if),   dWj_f += krho[t] (sum_i rh_if) xs_jf.
// step_base inversion steps were done before (several stages in a row keep counting); with MASKED the dW shares are
// weighted by `own` (1, or 0 for a group whose dW another window accounts for).
template <int NC, int EC, int R, int F, bool MASKED, bool TANH_ONLY = true, bool STEP_MASK = false, bool ROWS = false,
          bool KU_W = true>
__device__ __forceinline__ void headwise_backward_core(float (&Y)[R][F], float (&B)[R][F], float (&G)[R][F],
                                                       float (&P)[R][F], const float (&wi)[F], const float (&wj)[F],
                                                       float (&dwi)[F], float (&dwj)[F], float own, const StepTable& S,
                                                       int step_base, int lane, float4* slots, int live = NC) {
    using T = Tile<NC, EC, R, F>;
    const int rl = (lane / T::LF) % T::LR;
#pragma unroll 1
    for (int jo = T::LR - 1; jo >= 0; --jo) {
        const float selku = (T::LR == 1 || rl == jo) ? S.ku : 0.0f;  // this lane holds the pivot row
#pragma unroll
        for (int jr = R - 1; jr >= 0; --jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;
            const int ts = step_base + (T::LR - 1 - jo) * R + (R - 1 - jr);   // inversion steps done so far
            const float krho = MASKED ? S.krho[ts] * own : S.krho[ts];
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int f = 0; f < F; ++f) Y[rr][f] = fmaf(S.im, Y[rr][f], -B[rr][f]);  // xs before this step
            float xj[F], cj[F];
            row_lane_broadcast<T::LF, T::LR, F>(Y[jr], xj, jo, lane, slots);
#pragma unroll
            for (int f = 0; f < F; ++f) cj[f] = xj[f] * wj[f];
            if constexpr (T::LR == 1) {
                // The whole group is in this lane: every row's share of the pivot row's gradient,
                // ku (rh_if Wj'_f + c_if U_if) = ku U_if (xs_jf Wj'_f + c_if), goes straight into it, and dWj takes the
                // row's rh_if as dWi does (no sums to carry through the step: fewer registers).
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        const float c = fmaf(Y[rr][f], wi[f], cj[f]);
                        const float z = fmaf(c, xj[f], Y[rr][f]);
                        float w;
                        if constexpr (TANH_ONLY) {
                            const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
                            B[rr][f] = fmaf(S.bk1, r, fmaf(S.im, B[rr][f], S.bk0));   // bh before this step
                            w = fmaf(-r, r, r);
                        } else {
                            float Fv;
                            act_Fw(z, S.activation, Fv, w);
                            B[rr][f] = fmaf(S.bk0, Fv, S.im * B[rr][f]);
                        }
                        const float U = P[rr][f] * w;
                        const float rh = U * xj[f];
                        const float krh = krho * rh;
                        dwi[f] = fmaf(krh, Y[rr][f], dwi[f]);
                        dwj[f] = fmaf(krh, xj[f], dwj[f]);
                        G[rr][f] = fmaf(S.ku, fmaf(rh, wi[f], U), G[rr][f]);
                        G[jr][f] = fmaf(S.ku * U, cj[f] + c, G[jr][f]);
                        if (rr != jr) P[rr][f] = fmaf(S.om, G[rr][f], P[rr][f]);
                    }
                }
#pragma unroll
                for (int f = 0; f < F; ++f) P[jr][f] = fmaf(S.om, G[jr][f], P[jr][f]);
            } else {
            float v[F], rhs[F];
#pragma unroll
            for (int f = 0; f < F; ++f) v[f] = rhs[f] = 0.f;
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float c = fmaf(Y[rr][f], wi[f], cj[f]);
                    const float z = fmaf(c, xj[f], Y[rr][f]);
                    float w;
                    if constexpr (TANH_ONLY) {
                        const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
                        B[rr][f] = fmaf(S.bk1, r, fmaf(S.im, B[rr][f], S.bk0));   // bh before this step
                        w = fmaf(-r, r, r);
                    } else {
                        float Fv;
                        act_Fw(z, S.activation, Fv, w);
                        B[rr][f] = fmaf(S.bk0, Fv, S.im * B[rr][f]);
                    }
                    const float U = P[rr][f] * w;
                    const float rh = U * xj[f];
                    v[f] = fmaf(c, U, v[f]);
                    rhs[f] += rh;
                    dwi[f] = fmaf(krho * rh, Y[rr][f], dwi[f]);
                    G[rr][f] = fmaf(S.ku, fmaf(rh, wi[f], U), G[rr][f]);
                    if (rr != jr) P[rr][f] = fmaf(S.om, G[rr][f], P[rr][f]);
                }
            }
            float t[F];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                t[f] = fmaf(rhs[f], wj[f], v[f]);
                // every row lane of the group adds its share of sum_i rh_if: the sum over lanes at the end completes it
                dwj[f] = fmaf(krho * rhs[f], xj[f], dwj[f]);
            }
            lane_sum_n<T::LF, T::LPG, ROWS, F>(t);   // over the group's row lanes
#pragma unroll
            for (int f = 0; f < F; ++f) {
                G[jr][f] = fmaf(selku, t[f], G[jr][f]);
                P[jr][f] = fmaf(S.om, G[jr][f], P[jr][f]);
            }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

#define NCN_HW_PROLOGUE                                                                         \
    using T = Tile<NC, EC, R, F>;                                                               \
    const int lane = threadIdx.x & 63;                                                          \
    const int wave = threadIdx.x >> 6;                                                          \
    const uint32_t nwaves = gridDim.x * kWavesPerBlock;                                         \
    const uint32_t gwave = blockIdx.x * kWavesPerBlock + wave;                                  \
    const int head = gwave % A.n_head;                                                          \
    const uint32_t tile_step = nwaves / A.n_head;                                               \
    __shared__ float4 bcast_lds[T::LR == 1 ? 1 : kWavesPerBlock * (F / 4) * 64];                \
    float4* slots = bcast_lds + (T::LR == 1 ? 0 : wave * (F / 4) * 64);                         \
    const int fl = lane % T::LF;                                                                \
    float wi[F], wj[F];                                                                         \
    load_w<F>(A.W, A.E, head, EC, fl, wi, wj);                                                  \
    _Pragma("unroll") for (int f = 0; f < F; ++f) {                                             \
        wi[f] *= A.tab.gamma;                                                                   \
        wj[f] *= A.tab.gamma;                                                                   \
    }

#define NCN_HW_ROW_LIVE(rr) ((int)(((lane / T::LF) % T::LR) * R + (rr)) < live)

// rows past a context length, and the lanes of a wave tile past the last group: loaded from rows that exist, zeroed
// here, not stored
#define NCN_HW_ZERO_DEAD(p, q)                                                                  \
    if (__any(live != NC)) {                                                                    \
        _Pragma("unroll") for (int rr = 0; rr < R; ++rr) {                                      \
            const bool dead = !(INDEXED ? NCN_HW_ROW_LIVE(rr) : live != 0);                     \
            _Pragma("unroll") for (int f = 0; f < F; ++f) {                                     \
                p[rr][f] = dead ? 0.f : p[rr][f];                                               \
                q[rr][f] = dead ? 0.f : q[rr][f];                                               \
            }                                                                                   \
        }                                                                                       \
    }

// INVERSE = false: x, xa -> y, ya (optional float32 copies);  true: y, ya -> x, xa
template <int NC, int EC, int R, int F, bool TANH_ONLY, bool INDEXED, bool INVERSE>
__global__ void __launch_bounds__(kBlockThreads) headwise_forward_kernel(const StageArgs A) {
    NCN_HW_PROLOGUE
    for (uint32_t t = gwave / A.n_head; t < A.total_tiles; t += tile_step) {
        int64_t off[R];
        const int live = tile_offsets<NC, EC, R, F, INDEXED>(A, t, lane, head, off);
        float x[R][F], a[R][F];
        issue_tile<R, F>(A.in0, A.in_dtype, off, x, A.plane);
        issue_tile<R, F>(A.in1, A.in_dtype, off, a, A.plane);
        finish_tile<R, F>(A.in_dtype, x);
        finish_tile<R, F>(A.in_dtype, a);
        NCN_HW_ZERO_DEAD(x, a)
        if constexpr (INVERSE) {
            scale_tile<R, F>(x, a, A.tab.kappa, A.tab.b_scale);
            headwise_inverse_core<NC, EC, R, F, TANH_ONLY, INDEXED>(x, a, wi, wj, A.tab, lane, slots, live);
            scale_tile<R, F>(x, a, A.tab.inv_kappa, A.tab.inv_b_scale);
        } else {
            scale_tile<R, F>(x, a, A.tab.kappa, A.tab.a_scale);
            headwise_forward_core<NC, EC, R, F, TANH_ONLY, INDEXED>(x, a, wi, wj, A.tab, lane, slots, live);
            scale_tile<R, F>(x, a, A.tab.inv_kappa, A.tab.inv_a_scale);
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_HW_ROW_LIVE(rr) : live != 0;
            store_frag<F>(A.out0, A.out_dtype, off[rr], valid, x[rr], A.plane);
            store_frag<F>(A.out1, A.out_dtype, off[rr], valid, a[rr], A.plane);
            if (!INVERSE && A.aux0) {
                store_frag<F>(A.aux0, NCN_F32, off[rr], valid, x[rr]);
                store_frag<F>(A.aux1, NCN_F32, off[rr], valid, a[rr]);
            }
        }
    }
}

// LOOP = false is for launches with a wave for every tile, as in stage_backward_kernel: the build with the loop
// carries the tile's addresses across it and spills at R x F = 16.
template <int NC, int EC, int R, int F, bool TANH_ONLY, bool INDEXED, bool LOOP = true>
__global__ void __launch_bounds__(kBlockThreads, (TANH_ONLY && !INDEXED && R * F <= 16) ? 4 : 1) headwise_backward_kernel(const StageArgs A) {
    NCN_HW_PROLOGUE
    float dwi[F], dwj[F];
#pragma unroll
    for (int f = 0; f < F; ++f) dwi[f] = dwj[f] = 0.f;
    uint32_t t = gwave / A.n_head;
    if (t < A.total_tiles) do {
        int64_t off[R];
        const int live = tile_offsets<NC, EC, R, F, INDEXED>(A, t, lane, head, off);
        float Y[R][F], B[R][F], G[R][F], H[R][F];
        issue_tile<R, F>(A.in0, A.in_dtype, off, Y, A.plane);
        issue_tile<R, F>(A.in1, A.in_dtype, off, B, A.plane);
        issue_tile<R, F>(A.g0, A.g_dtype, off, G);
        if (A.g1) {
            issue_tile<R, F>(A.g1, A.g_dtype, off, H);
        } else {
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int f = 0; f < F; ++f) H[rr][f] = 0.f;
        }
        finish_tile<R, F>(A.in_dtype, Y);
        finish_tile<R, F>(A.in_dtype, B);
        finish_tile<R, F>(A.g_dtype, G);
        if (A.g1) finish_tile<R, F>(A.g_dtype, H);
        NCN_HW_ZERO_DEAD(Y, B)
        NCN_HW_ZERO_DEAD(G, H)
        // as if the NC - live skipped steps of a cut group had been done: G, P carry m^-t
        const float isc = (INDEXED && live != NC) ? pow_steps(A.tab.im, NC - live) : 1.0f;
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int f = 0; f < F; ++f) {
                Y[rr][f] *= A.tab.kappa;
                B[rr][f] *= A.tab.b_scale;
                H[rr][f] = fmaf(A.tab.om, G[rr][f], H[rr][f]);  // h -> p
                if (INDEXED) {
                    G[rr][f] *= isc;
                    H[rr][f] *= isc;
                }
            }
        headwise_backward_core<NC, EC, R, F, false, TANH_ONLY, INDEXED>(Y, B, G, H, wi, wj, dwi, dwj, 1.0f, A.tab, 0, lane, slots,
                                                                      live);
        const float dn = A.tab.m_pow_n;       // NC steps done: undo the scaling of the gradients
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
#pragma unroll
            for (int f = 0; f < F; ++f) {
                G[rr][f] *= dn;
                H[rr][f] = fmaf(H[rr][f], dn, -A.tab.om * G[rr][f]);  // back to h = p - (1-m) g
            }
            const bool valid = INDEXED ? NCN_HW_ROW_LIVE(rr) : live != 0;
            store_frag<F>(A.out0, A.out_dtype, off[rr], valid, G[rr]);
            store_frag<F>(A.out1, A.out_dtype, off[rr], valid, H[rr]);
            if (A.aux0) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    Y[rr][f] *= A.tab.inv_kappa;
                    B[rr][f] *= A.tab.inv_b_scale;
                }
                store_frag<F>(A.aux0, NCN_F32, off[rr], valid, Y[rr]);
                store_frag<F>(A.aux1, NCN_F32, off[rr], valid, B[rr]);
            }
        }
    } while (LOOP && (t += tile_step) < A.total_tiles);
    // dW: lanes holding the same features -> one value; this wave owns slot (gwave / n_head, head)
#pragma unroll
    for (int f = 0; f < F; ++f) {
        dwi[f] = lane_sum<T::LF, 64>(dwi[f]);
        dwj[f] = lane_sum<T::LF, 64>(dwj[f]);
    }
    if (lane < T::LF) {
        float* row = A.dw_partials + (int64_t)(gwave / A.n_head) * (2 * A.E) + (int64_t)head * EC + fl * F;
#pragma unroll
        for (int f = 0; f < F; ++f) {
            row[f] = dwi[f];
            row[A.E + f] = dwj[f];
        }
    }
}
#undef NCN_HW_PROLOGUE
#undef NCN_HW_ROW_LIVE
#undef NCN_HW_ZERO_DEAD

}  // namespace ncn
