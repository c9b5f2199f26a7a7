// Register-resident stage kernels: forward, inverse and reversible backward of ONE stage.
//
// Work decomposition.  A (batch, head, group) triple is an independent problem: n_cache rows of Ec
// features (torch_ref/ncn_pytorch.py:50-97).  Each lane keeps an R x F register tile of it: R
// consecutive rows of the group times F consecutive features of the head.  A row is thus spread
// over LF = Ec/F adjacent lanes and a group over LR = n_cache/R "row lanes" of LF lanes each, so
// one 64-wide wavefront carries 64/(LF*LR) whole groups ("a wave tile") and no step of the recurrence
// needs a workgroup barrier:
//   * the pivot row x_j of a step lives in row lane j/R, register row j%R; the other row lanes get
//     it through a wave-private LDS slot array (nothing to do when LR == 1),
//   * <x_i,Wi> + <x_j,Wj> and <u_i,x_j> are in-lane FMAs over F features plus log2(LF) DPP adds,
//   * the sum over rows that feeds the pivot row's gradient is an in-lane FMA chain over the R rows
//     plus log2(LR) cross-lane adds per feature register,
//   * <x_j,Wj> costs F FMAs per lane and step, i.e. 1/R per element.
// The step loop runs over j/R at run time and is unrolled over j%R, so register rows are addressed
// statically while the code stays R steps long.
// Wave w of the grid works on head w % n_head for its whole life (the grid holds a multiple of n_head
// waves) and loops over the wave tiles w / n_head, + waves / n_head, ..: the waves of a block therefore
// touch the n_head adjacent head slices of the same rows at about the same time, so a 128-byte line that
// holds two bf16 head slices is fetched from HBM once, not once per head.  A wave keeps its head's slices
// of Wi, Wj in registers, and in backward accumulates dWi, dWj in registers over all its tiles; they are
// reduced across its lanes once and leave as this wave's [2*Ec] slice of a partial row.
//
// Memory: a lane reads and writes only its own F-feature fragments of its own R rows (8/16-byte vector
// accesses; the LF lanes of a row cover its contiguous Ec-element head slice), each row exactly once
// per stage.
#pragma once
#include "ncn_device.h"

namespace ncn {

constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = 64 * kWavesPerBlock;

template <int NC, int EC, int R, int F>
struct Tile {
    static_assert(EC % F == 0 && NC % R == 0, "tile must divide the group");
    static constexpr int LF = EC / F;      // lanes per row
    static constexpr int LR = NC / R;      // row lanes per group
    static constexpr int LPG = LF * LR;    // lanes per group
    static_assert(LPG <= 64 && 64 % LPG == 0, "a group must fit one wavefront");
    static constexpr int GPW = 64 / LPG;   // groups per wave tile
    static constexpr int RLMASK = (LR - 1) * LF;
};

// Element offsets of this lane's R row fragments for wave tile `t`; returns the live rows of the lane's group:
// NC, or 0 when the group is past the end.  INDEXED builds read the grouping table and the context lengths when
// the launch has them (a group that a length cuts has 0 < live < NC); the plain builds only know the stride
// permutation (and are what every launch without table and lengths uses).
template <int NC, int EC, int R, int F, bool INDEXED>
__device__ __forceinline__ int tile_offsets(const StageArgs& A, uint32_t t, int lane, int head, int64_t (&off)[R]) {
    using T = Tile<NC, EC, R, F>;
    const int fl = lane % T::LF;
    const int rl = (lane / T::LF) % T::LR;
    const int gw = lane / T::LPG;
    const uint32_t b = t / A.tiles_per_inst;
    const uint32_t tile = t - b * A.tiles_per_inst;
    const uint32_t group = tile * T::GPW + gw;
    const bool valid = group < A.groups;
    const int live = !valid ? 0 : (INDEXED ? live_rows(A, b, group) : NC);
    const int64_t base = (int64_t)b * A.N * A.E + (int64_t)head * EC + fl * F;
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const uint32_t i = rl * R + rr;
        const int64_t pos = INDEXED ? slot_position(A, valid ? group : 0u, i)
                                    : (int64_t)stage_block(A, valid ? group : 0u, i) * NC + i;
        off[rr] = base + pos * A.E;
    }
    return live;
}

template <int F>
__device__ __forceinline__ void load_w(const float* W, int64_t E, int head, int ec, int fl, float (&wi)[F],
                                       float (&wj)[F]) {
    const float* w = W + (int64_t)head * ec + fl * F;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        wi[f] = w[f];
        wj[f] = w[E + f];
    }
}

// Activation from z = 2 log2(e) T (the form the step code produces): F(T) and w = F'(T) / 4.
//   tanh:    r = 1/(1 + 2^z), F = 1 - 2r, F'/4 = r - r^2                (ncn_fwd_cuda_kernel.cu:86-87)
//   relu, sigmoid, linear: codes of ncn_fwd_cuda_kernel.cu:88-95 / ncn_bwd_cuda_kernel.cu:137-150
// TANH_ONLY kernels never come here: their step code works on r itself.
constexpr float kHalfLn2 = 0.34657359027997264f;  // T = z * ln(2)/2
__device__ __forceinline__ void act_Fw(float z, int code, float& Fv, float& w) {
    if (code == NCN_ACT_TANH) {
        const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
        Fv = fmaf(-2.0f, r, 1.0f);
        w = fmaf(-r, r, r);
    } else if (code == NCN_ACT_RELU) {
        const float Tv = z * kHalfLn2;
        Fv = fmaxf(Tv, 0.f);
        w = Tv > 0.f ? 0.25f : 0.f;
    } else if (code == NCN_ACT_SIGMOID) {
        Fv = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(-0.5f * z) + 1.0f);
        w = 0.25f * fmaf(-Fv, Fv, Fv);
    } else if (code == NCN_ACT_LEAKY_RELU) {
        const float Tv = z * kHalfLn2;
        Fv = Tv >= 0.f ? Tv : 0.01f * Tv;
        w = Tv >= 0.f ? 0.25f : 0.0025f;
    } else {
        Fv = z * kHalfLn2;
        w = 0.25f;
    }
}

// The row sums c_i = <xs_i, Wi'> + <xs_j, Wj'> of a lane's R rows: a chain of FMAs per row that starts from the lane's
// share e of <xs_j, Wj'>, then all R sums cross the LF lanes of a row together.
template <int LF, int R, int F, bool ROWS>
__device__ __forceinline__ void row_sums(const float (&x)[R][F], const float (&wi)[F], float e, float (&c)[R]) {
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        c[rr] = e;
#pragma unroll
        for (int f = 0; f < F; ++f) c[rr] = fmaf(x[rr][f], wi[f], c[rr]);
    }
    lane_sum_n<1, LF, ROWS, R>(c);
}

template <int F>
__device__ __forceinline__ float dot_chain(const float (&a)[F], const float (&b)[F]) {
    float s = 0.f;
#pragma unroll
    for (int f = 0; f < F; ++f) s = fmaf(a[f], b[f], s);
    return s;
}

// ---------------------------------------------------------------------------------------------
// forward (torch_ref/ncn_pytorch.py:74-94), all n_cache steps on one register tile
//   s_i = <x_i,Wi> + <x_j,Wj>      T = alpha x_i + (1-alpha) s_i x_j      F = tanh T = 1 - 2r,
//   r = 1/(1 + exp(2T))            a' = m a + (1-m) F                     x' = m x + (1-m) a'
// on the scaled state of StepTable: x holds xs, a holds as, wi / wj hold gamma Wi / gamma Wj.  Per element and step:
// one FMA for the row sum, one for z, exp2, +1, rcp, two FMAs for as', one for xs'.
// STEP_MASK builds take `live`, the live rows of the lane's group, and skip steps j >= live with the lanes of that
// group switched off (a group that a context length cuts runs one step per live row,
// ncn_triton/ncn_triton_old.py:93-96).  Every cross-lane exchange of a step stays inside one group.
// ---------------------------------------------------------------------------------------------
template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void forward_core(float (&x)[R][F], float (&a)[R][F], const float (&wi)[F],
                                             const float (&wj)[F], const StepTable& S, int lane, float4* slots,
                                             int live = NC) {
    using T = Tile<NC, EC, R, F>;
#pragma unroll 1
    for (int jo = 0; jo < T::LR; ++jo) {
#pragma unroll
        for (int jr = 0; jr < R; ++jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;  // the lanes of a group agree: no lane it needs is off
            float xj[F], c[R];
            row_lane_broadcast<T::LF, T::LR, F>(x[jr], xj, jo, lane, slots);
            row_sums<T::LF, R, F, ROWS>(x, wi, dot_chain<F>(xj, wj), c);
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float z = fmaf(c[rr], xj[f], x[rr][f]);
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

// ---------------------------------------------------------------------------------------------
// inverse (torch_ref/ncn_pytorch_invertible.py:87-113), steps j = n_cache-1 .. 0
//   x = (y - (1-m) b)/m       recompute r from x        a = (b - (1-m) F)/m
// on the scaled state: y holds xs, b holds bh (see StepTable).
// STEP_MASK: a group with `live` < NC live rows only undoes its steps live-1 .. 0.
// ---------------------------------------------------------------------------------------------
template <int NC, int EC, int R, int F, bool TANH_ONLY, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void inverse_core(float (&y)[R][F], float (&b)[R][F], const float (&wi)[F],
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
            float xj[F], c[R];
            row_lane_broadcast<T::LF, T::LR, F>(y[jr], xj, jo, lane, slots);
            row_sums<T::LF, R, F, ROWS>(y, wi, dot_chain<F>(xj, wj), c);
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float z = fmaf(c[rr], xj[f], y[rr][f]);
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

// ---------------------------------------------------------------------------------------------
// reversible backward: per step, invert (ncn_bwd_cuda_kernel.cu:88-115), then the closed-form
// vector-Jacobian product (vectorised statement: ncn_triton/ncn_triton.py:198-246).  With g = dL/dx',
// h = dL/da' and p = (1-m) g + h carried instead of h:
//   u_i  = (1-m) p_i F'(T_i),   F' = 1 - F^2 = 4 r (1 - r)          r_i = <u_i, x_j>
//   dWi += (1-a) r_i x_i        dWj += (1-a) (sum_i r_i) x_j
//   g_i <- m g_i + a u_i + (1-a) r_i Wi   [+ sum_k ((1-a) r_k Wj + (1-a) s_k u_k) on the pivot row j]
//   p_i <- (1-m) g_i(new) + m p_i          (equivalent to h_i <- m (1-m) g_i + m h_i)
//
// Registers: Y = xs, B = bh (scaled state, see StepTable), G = g / m^t, P = p / m^t after t inversion steps, which
// turns  g <- m g + ..  into  G <- G + ../m^(t+1)  and  p <- (1-m) g + m p  into  P <- P + (1-m) G  (one FMA each).
// With U = P F'/4 (so u = 4 (1-m) m^t U) and rh_i = <U_i, xs_j> every factor that is not a power of m is the one
// constant ku = 4 (1-m) alpha / m:
//   G_i += ku (U_i + rh_i Wi')           pivot row: G_j += ku sum_rows( (sum_i rh_i) Wj' + sum_i c_i U_i )
// and only dW needs the true scale: dWi += krho[t] rh_i xs_i, dWj += krho[t] (sum_i rh_i) xs_j.
//
// A step runs in phases over the lane's R rows, so that the cross-lane sums of the rows travel together:
// invert xs; row sums c; [per element: z, r, bh, U, partial rh, v += c U, G += ku U]; sums rh; [G += ku rh Wi', dWi, P];
// pivot row.  U is only needed inside the third phase.
//
// On entry Y, B = scaled stage outputs, G = g / m^t0, P = p / m^t0 with t0 = step_base inversion steps done before
// (several stages in a row keep counting); on exit all four describe the stage inputs, t0 + n_cache steps done.
// dwi, dwj accumulate this lane's share of dWi, dWj; with MASKED the share is weighted by `own` (1, or 0 for a
// group whose dW another tile accounts for).
// STEP_MASK: steps j >= live leave the registers as they are (the caller scales G, P as if they had been done).
// ---------------------------------------------------------------------------------------------
// KU_W: the products ku Wi' are kept beside the weights (F more registers, one multiplication less per row and step).
template <int NC, int EC, int R, int F, bool MASKED, bool TANH_ONLY = true, bool STEP_MASK = false, bool ROWS = false,
          bool KU_W = true>
__device__ __forceinline__ void backward_core(float (&Y)[R][F], float (&B)[R][F], float (&G)[R][F], float (&P)[R][F],
                                              const float (&wi)[F], const float (&wj)[F], float (&dwi)[F],
                                              float (&dwj)[F], float own, const StepTable& S, int step_base, int lane,
                                              float4* slots, int live = NC) {
    using T = Tile<NC, EC, R, F>;
    const int rl = (lane / T::LF) % T::LR;
    float wiku[KU_W ? F : 1];   // ku Wi': G += rh (ku Wi') spares the product ku rh of every row and step
    if constexpr (KU_W) {
#pragma unroll
        for (int f = 0; f < F; ++f) wiku[f] = S.ku * wi[f];
    }
#pragma unroll 1
    for (int jo = T::LR - 1; jo >= 0; --jo) {
        const float selku = (T::LR == 1 || rl == jo) ? S.ku : 0.0f;  // this lane holds the pivot row
#pragma unroll
        for (int jr = R - 1; jr >= 0; --jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;  // lanes of a group agree: no lane it needs is off
            const int ts = step_base + (T::LR - 1 - jo) * R + (R - 1 - jr);   // inversion steps done so far
            const float krho = MASKED ? S.krho[ts] * own : S.krho[ts];
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int f = 0; f < F; ++f) Y[rr][f] = fmaf(S.im, Y[rr][f], -B[rr][f]);  // xs before this step
            float xj[F], c[R], rh[R];
            row_lane_broadcast<T::LF, T::LR, F>(Y[jr], xj, jo, lane, slots);
            row_sums<T::LF, R, F, ROWS>(Y, wi, dot_chain<F>(xj, wj), c);
            if constexpr (T::LR == 1) {
                // The whole group is in this lane: the pivot row's share sum_i c_i U_i goes straight into its gradient
                // (no sum across lanes to wait for), with the pivot's own two terms merged into one coefficient.
                float kc[R];
#pragma unroll
                for (int rr = 0; rr < R; ++rr) kc[rr] = (rr == jr) ? fmaf(S.ku, c[rr], S.ku) : S.ku * c[rr];
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    rh[rr] = 0.f;
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        const float z = fmaf(c[rr], xj[f], Y[rr][f]);
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
                        rh[rr] = fmaf(U, xj[f], rh[rr]);
                        if (rr != jr) G[rr][f] = fmaf(S.ku, U, G[rr][f]);
                        G[jr][f] = fmaf(kc[rr], U, G[jr][f]);
                    }
                }
                lane_sum_n<1, T::LF, ROWS, R>(rh);
                float rhosum = 0.f;
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    const float rho_w = krho * rh[rr];     // (1-alpha) r_i / kappa, weighted
                    const float rho_ku = KU_W ? rh[rr] : S.ku * rh[rr];
                    rhosum += rh[rr];
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        dwi[f] = fmaf(rho_w, Y[rr][f], dwi[f]);
                        G[rr][f] = fmaf(rho_ku, KU_W ? wiku[f] : wi[f], G[rr][f]);
                    }
                }
                const float rhosum_w = krho * rhosum, rhosum_ku = S.ku * rhosum;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    dwj[f] = fmaf(rhosum_w, xj[f], dwj[f]);
                    G[jr][f] = fmaf(rhosum_ku, wj[f], G[jr][f]);
                }
#pragma unroll
                for (int rr = 0; rr < R; ++rr)
#pragma unroll
                    for (int f = 0; f < F; ++f) P[rr][f] = fmaf(S.om, G[rr][f], P[rr][f]);
            } else {
            float v[F];
#pragma unroll
            for (int f = 0; f < F; ++f) v[f] = 0.f;
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                rh[rr] = 0.f;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float z = fmaf(c[rr], xj[f], Y[rr][f]);
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
                    rh[rr] = fmaf(U, xj[f], rh[rr]);
                    v[f] = fmaf(c[rr], U, v[f]);
                    G[rr][f] = fmaf(S.ku, U, G[rr][f]);
                }
            }
            lane_sum_n<1, T::LF, ROWS, R>(rh);
            float rhosum = 0.f;
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const float rho_w = krho * rh[rr];     // (1-alpha) r_i / kappa, weighted
                const float rho_ku = KU_W ? rh[rr] : S.ku * rh[rr];
                rhosum += rh[rr];
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    dwi[f] = fmaf(rho_w, Y[rr][f], dwi[f]);
                    G[rr][f] = fmaf(rho_ku, KU_W ? wiku[f] : wi[f], G[rr][f]);
                    if (rr != jr) P[rr][f] = fmaf(S.om, G[rr][f], P[rr][f]);
                }
            }
            const float rhosum_w = krho * rhosum;
            float t[F];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                dwj[f] = fmaf(rhosum_w, xj[f], dwj[f]);
                t[f] = fmaf(rhosum, wj[f], v[f]);
            }
            lane_sum_n<T::LF, T::LPG, ROWS, F>(t);   // over the group's row lanes
#pragma unroll
            for (int f = 0; f < F; ++f) {
                G[jr][f] = fmaf(selku, t[f], G[jr][f]);
                P[jr][f] = fmaf(S.om, G[jr][f], P[jr][f]);
            }
            }
            __builtin_amdgcn_sched_barrier(0);  // keep steps apart: interleaving them only costs registers
        }
    }
}

// m^k by repeated multiplication (k <= 64; only groups cut by a context length come here)
__device__ __forceinline__ float pow_steps(float base, int k) {
    float p = 1.0f;
    for (int i = 0; i < k; ++i) p *= base;
    return p;
}

// True values <-> scaled state, on a register tile.
template <int R, int F>
__device__ __forceinline__ void scale_tile(float (&x)[R][F], float (&a)[R][F], float sx, float sa) {
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) {
            x[rr][f] *= sx;
            a[rr][f] *= sa;
        }
}

// one stage of the backward from true values to true values: G, H true gradients in and out; Y, B true outputs in,
// true inputs out
template <int NC, int EC, int R, int F, bool MASKED, bool TANH_ONLY, bool STEP_MASK = false>
__device__ __forceinline__ void backward_steps(float (&Y)[R][F], float (&B)[R][F], float (&G)[R][F], float (&P)[R][F],
                                               const float (&wi)[F], const float (&wj)[F], float (&dwi)[F],
                                               float (&dwj)[F], float own, const StepTable& S, int lane,
                                               float4* slots, int live = NC) {
    // as if the NC - live skipped steps of a cut group had been done: G, P carry m^-t
    const float isc = (STEP_MASK && live != NC) ? pow_steps(S.im, NC - live) : 1.0f;
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) {
            Y[rr][f] *= S.kappa;
            B[rr][f] *= S.b_scale;
            P[rr][f] = fmaf(S.om, G[rr][f], P[rr][f]);  // h -> p
            if (STEP_MASK) {
                G[rr][f] *= isc;
                P[rr][f] *= isc;
            }
        }
    backward_core<NC, EC, R, F, MASKED, TANH_ONLY, STEP_MASK>(Y, B, G, P, wi, wj, dwi, dwj, own, S, 0, lane, slots,
                                                             live);
    const float dn = S.m_pow_n;       // NC steps done: undo the scaling of the gradients
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) {
            G[rr][f] *= dn;
            P[rr][f] = fmaf(P[rr][f], dn, -S.om * G[rr][f]);  // back to h = p - (1-m) g
        }
}

// ---------------------------------------------------------------------------------------------
// One-stage kernels: gather the register tile from HBM, run the steps, scatter.
// ---------------------------------------------------------------------------------------------
#define NCN_WAVE_PROLOGUE                                                                       \
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
    bool w_raw = true;

// The weights are scaled by gamma once, after the loads of the wave's first tile have been issued: scaling them in the
// prologue would wait for them before the tile's own loads are even on their way (one memory latency after the other).
#define NCN_SCALE_W_ONCE                                                                        \
    if (w_raw) {                                                                                \
        w_raw = false;                                                                          \
        _Pragma("unroll") for (int f = 0; f < F; ++f) {                                         \
            wi[f] *= A.tab.gamma;                                                               \
            wj[f] *= A.tab.gamma;                                                               \
        }                                                                                       \
    }

// Row rr of this lane is live when its slot is below the group's live rows (always, or never, without lengths).
#define NCN_ROW_LIVE(rr) ((int)(((lane / T::LF) % T::LR) * R + (rr)) < live)

// Tiles are loaded without predicates (the offsets of lanes and rows without work point at rows that exist): rows past
// a context length, and the lanes of a wave tile past the last group, are zeroed here, so that they add nothing to the
// sums of their group or to dW.  Most wave tiles have no such rows: with `skip`, one wave-uniform branch jumps over
// the selects (1.7 % on the forward; the backward, whose registers are tighter, is no faster for it).
#define NCN_ZERO_DEAD_ROWS(p, q, skip)                                                          \
    if (!(skip) || __any(live != NC)) {                                                         \
        _Pragma("unroll") for (int rr = 0; rr < R; ++rr) {                                      \
            const bool dead = !(INDEXED ? NCN_ROW_LIVE(rr) : live != 0);                        \
            _Pragma("unroll") for (int f = 0; f < F; ++f) {                                     \
                p[rr][f] = dead ? 0.f : p[rr][f];                                               \
                q[rr][f] = dead ? 0.f : q[rr][f];                                               \
            }                                                                                   \
        }                                                                                       \
    }

template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool INDEXED = false>
__global__ void __launch_bounds__(kBlockThreads, (TANH_ONLY && !INDEXED && R == 4 && F == 4) ? 5 : 1) stage_forward_kernel(const StageArgs A) {
    NCN_WAVE_PROLOGUE
    for (uint32_t t = gwave / A.n_head; t < A.total_tiles; t += tile_step) {
        int64_t off[R];
        const int live = tile_offsets<NC, EC, R, F, INDEXED>(A, t, lane, head, off);
        float x[R][F], a[R][F];
        issue_tile<R, F>(A.in0, A.in_dtype, off, x);
        issue_tile<R, F>(A.in1, A.in_dtype, off, a);
        NCN_SCALE_W_ONCE
        finish_tile<R, F>(A.in_dtype, x);
        finish_tile<R, F>(A.in_dtype, a);
        NCN_ZERO_DEAD_ROWS(x, a, true)
        scale_tile<R, F>(x, a, A.tab.kappa, A.tab.a_scale);
        forward_core<NC, EC, R, F, TANH_ONLY, INDEXED>(x, a, wi, wj, A.tab, lane, slots, live);
        scale_tile<R, F>(x, a, A.tab.inv_kappa, A.tab.inv_a_scale);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            store_frag<F>(A.out0, A.out_dtype, off[rr], valid, x[rr], A.plane);
            store_frag<F>(A.out1, A.out_dtype, off[rr], valid, a[rr], A.plane);
            if (A.aux0) {
                store_frag<F>(A.aux0, NCN_F32, off[rr], valid, x[rr]);
                store_frag<F>(A.aux1, NCN_F32, off[rr], valid, a[rr]);
            }
        }
    }
}

template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool INDEXED = false>
__global__ void __launch_bounds__(kBlockThreads) stage_inverse_kernel(const StageArgs A) {
    NCN_WAVE_PROLOGUE
    for (uint32_t t = gwave / A.n_head; t < A.total_tiles; t += tile_step) {
        int64_t off[R];
        const int live = tile_offsets<NC, EC, R, F, INDEXED>(A, t, lane, head, off);
        float y[R][F], b[R][F];
        issue_tile<R, F>(A.in0, A.in_dtype, off, y, A.plane);
        issue_tile<R, F>(A.in1, A.in_dtype, off, b, A.plane);
        NCN_SCALE_W_ONCE
        finish_tile<R, F>(A.in_dtype, y);
        finish_tile<R, F>(A.in_dtype, b);
        NCN_ZERO_DEAD_ROWS(y, b, true)
        scale_tile<R, F>(y, b, A.tab.kappa, A.tab.b_scale);
        inverse_core<NC, EC, R, F, TANH_ONLY, INDEXED>(y, b, wi, wj, A.tab, lane, slots, live);
        scale_tile<R, F>(y, b, A.tab.inv_kappa, A.tab.inv_b_scale);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            store_frag<F>(A.out0, A.out_dtype, off[rr], valid, y[rr]);
            store_frag<F>(A.out1, A.out_dtype, off[rr], valid, b[rr]);
        }
    }
}

// Tiles of up to 16 elements per lane fit 128 VGPRs (4 waves per SIMD) when the compiler is asked to.  Larger tiles,
// the multi-activation build and the builds that mask steps would spill, so they are left alone.
// LOOP = false is for launches with a wave for every tile: without the loop around them the tile's addresses and
// offsets are not carried in registers across it (the loop build spills 6 of them per lane at R x F = 16, which a
// launch bound by its traffic pays for), and the steps come out in an order that issues better.
template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool INDEXED = false, bool LOOP = true>
__global__ void __launch_bounds__(kBlockThreads, (TANH_ONLY && R * F <= 16 && F == 4) ? 4 : 1) stage_backward_kernel(const StageArgs A) {
    NCN_WAVE_PROLOGUE
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
        NCN_SCALE_W_ONCE
        finish_tile<R, F>(A.in_dtype, Y);
        finish_tile<R, F>(A.in_dtype, B);
        finish_tile<R, F>(A.g_dtype, G);
        if (A.g1) finish_tile<R, F>(A.g_dtype, H);
        NCN_ZERO_DEAD_ROWS(Y, B, false)
        NCN_ZERO_DEAD_ROWS(G, H, false)
        backward_steps<NC, EC, R, F, false, TANH_ONLY, INDEXED>(Y, B, G, H, wi, wj, dwi, dwj, 1.0f, A.tab, lane, slots,
                                                               live);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
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

    // dW: lanes holding the same feature chunk -> one value; this wave owns slot (gwave / n_head, head).
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
#undef NCN_ROW_LIVE
#undef NCN_ZERO_DEAD_ROWS
#undef NCN_SCALE_W_ONCE
#undef NCN_WAVE_PROLOGUE

}  // namespace ncn
