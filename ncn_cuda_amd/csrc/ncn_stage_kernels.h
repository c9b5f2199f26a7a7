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
constexpr float kTwoLog2e = 2.8853900817779268f;  // exp(2T) = exp2(kTwoLog2e * T)

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
// TANH_ONLY kernels have no branch; the others pick the activation with a wave-uniform branch on `code`.
constexpr float kHalfLn2 = 0.34657359027997264f;  // T = z * ln(2)/2
template <bool TANH_ONLY>
__device__ __forceinline__ void act_Fw(float z, int code, float& Fv, float& w) {
    if (TANH_ONLY || code == NCN_ACT_TANH) {
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

template <int F>
__device__ __forceinline__ float dot_frag(const float (&a)[F], const float (&b)[F]) {
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int f = 0; f < F; f += 2) {
        s0 = fmaf(a[f], b[f], s0);
        if (f + 1 < F) s1 = fmaf(a[f + 1], b[f + 1], s1);
    }
    return s0 + s1;
}

// ---------------------------------------------------------------------------------------------
// forward (torch_ref/ncn_pytorch.py:74-94), all n_cache steps on one register tile
//   s_i = <x_i,Wi> + <x_j,Wj>      T = alpha x_i + (1-alpha) s_i x_j      F = tanh T = 1 - 2r,
//   r = 1/(1 + exp(2T))            a' = m a + (1-m) F                     x' = m x + (1-m) a'
// The registers hold X = x / m^t and A = xa / m^t after t steps, which turns the two updates into
//   A <- A + (1-m)/m^(t+1) F   and   X <- X + (1-m) A   (the powers of m come from a host-made table).
// ---------------------------------------------------------------------------------------------
// forward_core runs the n_cache steps of one stage on registers that already hold x / m^t0, xa / m^t0 with
// t0 = step_base steps done before (several stages in a row just keep counting) and leaves them scaled.
// STEP_MASK builds take `live`, the live rows of the lane's group, and skip steps j >= live with the lanes of that
// group switched off (a group that a context length cuts runs one step per live row,
// ncn_triton/ncn_triton_old.py:93-96).  Every cross-lane exchange of a step stays inside one group.
template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void forward_core(float (&x)[R][F], float (&a)[R][F], const float (&wi)[F],
                                             const float (&wj)[F], const StepTable& S, int step_base, int lane,
                                             float4* slots, int live = NC) {
    using T = Tile<NC, EC, R, F>;
    const float om = 1.0f - S.m;
#pragma unroll 1
    for (int jo = 0; jo < T::LR; ++jo) {
#pragma unroll
        for (int jr = 0; jr < R; ++jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;  // the lanes of a group agree: no lane it needs is off
            const int ts = step_base + jo * R + jr;   // steps done so far
            const float lam = S.step[ts].flam;     // z = lam X_i + c_i Xj
            const float kc = S.step[ts].fkc;       // c_i = kc S_i
            const float kap = S.step[ts].fkap;     // A <- A + kap F
            float xj[F];
            row_lane_broadcast<T::LF, T::LR, F>(x[jr], xj, jo, lane, slots);
            const float e = dot_frag<F>(xj, wj);
            // pivot row last: its registers are the source of xj when LR == 1
#pragma unroll
            for (int k = 1; k <= R; ++k) {
                const int rr = (jr + k) % R;
                const float s = lane_sum<1, T::LF, ROWS>(dot_frag<F>(x[rr], wi) + e);
                const float c = kc * s;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float z = fmaf(c, xj[f], lam * x[rr][f]);
                    float Fv, w;
                    act_Fw<TANH_ONLY>(z, S.activation, Fv, w);
                    a[rr][f] = fmaf(kap, Fv, a[rr][f]);
                    x[rr][f] = fmaf(om, a[rr][f], x[rr][f]);
                }
            }
        }
    }
}

// one stage from true values to true values
// m^k by repeated multiplication (k <= 64; only groups cut by a context length come here)
__device__ __forceinline__ float pow_steps(float base, int k) {
    float p = 1.0f;
    for (int i = 0; i < k; ++i) p *= base;
    return p;
}

template <int NC, int EC, int R, int F, bool TANH_ONLY, bool STEP_MASK = false>
__device__ __forceinline__ void forward_steps(float (&x)[R][F], float (&a)[R][F], const float (&wi)[F],
                                              const float (&wj)[F], const StepTable& S, int lane, float4* slots,
                                              int live = NC) {
    forward_core<NC, EC, R, F, TANH_ONLY, STEP_MASK>(x, a, wi, wj, S, 0, lane, slots, live);
    // `live` steps were done: the registers hold x / m^live
    const float dn = (!STEP_MASK || live == NC) ? S.m_pow_n : pow_steps(S.m, live);
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) {
            x[rr][f] *= dn;
            a[rr][f] *= dn;
        }
}

// ---------------------------------------------------------------------------------------------
// inverse (torch_ref/ncn_pytorch_invertible.py:87-113), steps j = n_cache-1 .. 0
//   x = (y - (1-m) b)/m       recompute r from x        a = (b - (1-m) F)/m
// with the same m^t scaling of the registers as the backward below (Y = m^t x, B = m^t xa).
// ---------------------------------------------------------------------------------------------
// STEP_MASK: a group with `live` < NC live rows only undoes its steps live-1 .. 0.  The skipped steps come first in
// the loop, so the registers are first scaled as if they had been done (m^(NC-live)): every later step then
// finds the scaling its table entry assumes, and the final factor is the same for all groups.
// inverse_core: the n_cache steps of one stage on registers that hold m^t0 x, m^t0 xa with t0 = step_base inversion
// steps done before; leaves them scaled by t0 + n_cache steps (several stages in a row just keep counting).
template <int NC, int EC, int R, int F, bool TANH_ONLY, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void inverse_core(float (&y)[R][F], float (&b)[R][F], const float (&wi)[F],
                                             const float (&wj)[F], const StepTable& S, int step_base, int lane,
                                             float4* slots, int live = NC) {
    using T = Tile<NC, EC, R, F>;
    const float nom = S.m - 1.0f;
#pragma unroll 1
    for (int jo = T::LR - 1; jo >= 0; --jo) {
#pragma unroll
        for (int jr = R - 1; jr >= 0; --jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;
            const int ts = step_base + (T::LR - 1 - jo) * R + (R - 1 - jr);   // inversion steps done so far
            const float lam = S.step[ts].lam, kc2 = S.step[ts].kc2, kap = S.step[ts].kap;
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int f = 0; f < F; ++f) y[rr][f] = fmaf(nom, b[rr][f], y[rr][f]);
            float xj[F];
            row_lane_broadcast<T::LF, T::LR, F>(y[jr], xj, jo, lane, slots);
            const float e = dot_frag<F>(xj, wj);
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const float s = lane_sum<1, T::LF, ROWS>(dot_frag<F>(y[rr], wi) + e);
                const float c = kc2 * s;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float z = fmaf(c, xj[f], lam * y[rr][f]);
                    float Fv, w;
                    act_Fw<TANH_ONLY>(z, S.activation, Fv, w);
                    b[rr][f] = fmaf(-kap, Fv, b[rr][f]);
                }
            }
        }
    }
}

// one stage from true values to true values
template <int NC, int EC, int R, int F, bool TANH_ONLY, bool STEP_MASK = false>
__device__ __forceinline__ void inverse_steps(float (&y)[R][F], float (&b)[R][F], const float (&wi)[F],
                                              const float (&wj)[F], const StepTable& S, int lane, float4* slots,
                                              int live = NC) {
    if (STEP_MASK && live != NC) {
        const float sc = pow_steps(S.m, NC - live);
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int f = 0; f < F; ++f) {
                y[rr][f] *= sc;
                b[rr][f] *= sc;
            }
    }
    inverse_core<NC, EC, R, F, TANH_ONLY, STEP_MASK>(y, b, wi, wj, S, 0, lane, slots, live);
    const float up = S.inv_m_pow_n;
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) {
            y[rr][f] *= up;
            b[rr][f] *= up;
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
// The divisions by m of the inversion and the multiplications by m of the gradient recurrences are
// folded into per-step scalars: after t inversion steps the registers hold
//   Y = m^t x,   B = m^t xa,   G = g / m^t,   P = p / m^t,
// which turns  x <- (y - (1-m) b)/m  into  Y <- Y - (1-m) B,   g <- m g + ..  into  G <- G + ../m^(t+1)
// and  p <- (1-m) g + m p  into  P <- P + (1-m) G  (one FMA each).
//
// On entry Y, B = stage outputs, G, H = their gradients; on exit G, H = gradients of the stage inputs and
// Y, B = m^n_cache times the stage inputs (multiply by StepTable::inv_m_pow_n before storing them).
// dwi, dwj accumulate this lane's share of dWi, dWj; with MASKED the share is weighted by `own` (1, or 0 for a
// group whose dW another tile accounts for).
// ---------------------------------------------------------------------------------------------
// backward_core: the n_cache steps of one stage on registers in the scaled form above with t0 = step_base
// inversion steps done before (P holds p / m^t0, not h); leaves them scaled by t0 + n_cache steps.
// STEP_MASK: steps j >= live leave the registers as they are (see inverse_steps for the scaling).
template <int NC, int EC, int R, int F, bool MASKED, bool TANH_ONLY = true, bool STEP_MASK = false, bool ROWS = false>
__device__ __forceinline__ void backward_core(float (&Y)[R][F], float (&B)[R][F], float (&G)[R][F], float (&P)[R][F],
                                              const float (&wi)[F], const float (&wj)[F], float (&dwi)[F],
                                              float (&dwj)[F], float own, const StepTable& S, int step_base, int lane,
                                              float4* slots, int live = NC) {
    using T = Tile<NC, EC, R, F>;
    const int rl = (lane / T::LF) % T::LR;
    const float om = 1.0f - S.m;
    const float ku = 4.0f * om / S.m * S.alpha;  // G += ku * U        (U = P (r - r^2))
    const float nom = -om;
#pragma unroll 1
    for (int jo = T::LR - 1; jo >= 0; --jo) {
        const float sel = (T::LR == 1 || rl == jo) ? 1.0f : 0.0f;  // this lane holds the pivot row
#pragma unroll
        for (int jr = R - 1; jr >= 0; --jr) {
            if (STEP_MASK && jo * R + jr >= live) continue;  // lanes of a group agree: no lane it needs is off
            const int ts = step_base + (T::LR - 1 - jo) * R + (R - 1 - jr);   // inversion steps done so far
            const float lam = S.step[ts].lam;     // z = lam Y_i + chat_i Yj
            const float kc2 = S.step[ts].kc2;     // chat_i = kc2 S_i
            const float kap = S.step[ts].kap;     // B <- B - kap F
            const float krho = S.step[ts].krho;   // rho_i = krho <U_i, Yj>
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int f = 0; f < F; ++f) Y[rr][f] = fmaf(nom, B[rr][f], Y[rr][f]);  // m^(t+1) x of this step
            float xj[F], v[F];
            row_lane_broadcast<T::LF, T::LR, F>(Y[jr], xj, jo, lane, slots);
#pragma unroll
            for (int f = 0; f < F; ++f) v[f] = 0.f;
            const float e = dot_frag<F>(xj, wj);
            float rhosum = 0.f;
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const float Ssum = lane_sum<1, T::LF, ROWS>(dot_frag<F>(Y[rr], wi) + e);
                const float chat = kc2 * Ssum;
                float u[F];
                float rh = 0.f;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    const float z = fmaf(chat, xj[f], lam * Y[rr][f]);
                    float Fv, w;
                    act_Fw<TANH_ONLY>(z, S.activation, Fv, w);
                    B[rr][f] = fmaf(-kap, Fv, B[rr][f]);   // m^(t+1) xa of this step
                    u[f] = P[rr][f] * w;
                    rh = fmaf(u[f], xj[f], rh);
                }
                rh = lane_sum<1, T::LF, ROWS>(rh);
                const float rho = krho * rh;       // (1-alpha) r_i / m^(t+1)
                const float c4 = krho * Ssum;      // (1-alpha) s_i u-scale / m^(t+1)
                const float rho_w = MASKED ? rho * own : rho;
                rhosum += rho;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    dwi[f] = fmaf(rho_w, Y[rr][f], dwi[f]);
                    v[f] = fmaf(c4, u[f], v[f]);
                    G[rr][f] = fmaf(rho, wi[f], fmaf(ku, u[f], G[rr][f]));
                    if (rr != jr) P[rr][f] = fmaf(om, G[rr][f], P[rr][f]);
                }
            }
            const float rhosum_w = MASKED ? rhosum * own : rhosum;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                dwj[f] = fmaf(rhosum_w, xj[f], dwj[f]);
                const float vt = lane_sum<T::LF, T::LPG, ROWS>(fmaf(rhosum, wj[f], v[f]));  // over the group's row lanes
                G[jr][f] = fmaf(sel, vt, G[jr][f]);
                P[jr][f] = fmaf(om, G[jr][f], P[jr][f]);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep steps apart: interleaving them only costs registers
        }
    }
}

// one stage: G, H true gradients in and out; Y, B true outputs in, m^n_cache times the stage inputs out
template <int NC, int EC, int R, int F, bool MASKED, bool TANH_ONLY, bool STEP_MASK = false>
__device__ __forceinline__ void backward_steps(float (&Y)[R][F], float (&B)[R][F], float (&G)[R][F], float (&P)[R][F],
                                               const float (&wi)[F], const float (&wj)[F], float (&dwi)[F],
                                               float (&dwj)[F], float own, const StepTable& S, int lane,
                                               float4* slots, int live = NC) {
    const float om = 1.0f - S.m;
    const float nom = -om;
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) P[rr][f] = fmaf(om, G[rr][f], P[rr][f]);  // h -> p
    if (STEP_MASK && live != NC) {
        // as if the NC - live skipped steps had been done: Y, B carry m^t, G, P carry m^-t
        const float sc = pow_steps(S.m, NC - live), isc = pow_steps(1.0f / S.m, NC - live);
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int f = 0; f < F; ++f) {
                Y[rr][f] *= sc;
                B[rr][f] *= sc;
                G[rr][f] *= isc;
                P[rr][f] *= isc;
            }
    }
    backward_core<NC, EC, R, F, MASKED, TANH_ONLY, STEP_MASK>(Y, B, G, P, wi, wj, dwi, dwj, own, S, 0, lane, slots,
                                                             live);
    // undo the scaling of the gradients: NC steps done
    const float dn = S.m_pow_n;       // m^NC
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int f = 0; f < F; ++f) {
            G[rr][f] *= dn;
            P[rr][f] = fmaf(P[rr][f], dn, nom * G[rr][f]);  // back to h = p - (1-m) g
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
    load_w<F>(A.W, A.E, head, EC, fl, wi, wj);

// Row rr of this lane is live when its slot is below the group's live rows (always, or never, without lengths).
#define NCN_ROW_LIVE(rr) ((int)(((lane / T::LF) % T::LR) * R + (rr)) < live)

// The 4 x 4 tanh build fits 72 VGPRs (7 waves per SIMD) when asked to, against the 78 (6 waves) the compiler picks by
// itself: measured 5 % faster on the headline shape (a wave issues more often with more waves to pick from).  The
// other builds would spill.
template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool INDEXED = false>
__global__ void __launch_bounds__(kBlockThreads, (TANH_ONLY && !INDEXED && R == 4 && F == 4) ? 7 : 1) stage_forward_kernel(const StageArgs A) {
    NCN_WAVE_PROLOGUE
    for (uint32_t t = gwave / A.n_head; t < A.total_tiles; t += tile_step) {
        int64_t off[R];
        const int live = tile_offsets<NC, EC, R, F, INDEXED>(A, t, lane, head, off);
        float x[R][F], a[R][F];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            load_frag<F>(A.in0, A.in_dtype, off[rr], valid, x[rr]);
            load_frag<F>(A.in1, A.in_dtype, off[rr], valid, a[rr]);
        }
        forward_steps<NC, EC, R, F, TANH_ONLY, INDEXED>(x, a, wi, wj, A.tab, lane, slots, live);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            store_frag<F>(A.out0, A.out_dtype, off[rr], valid, x[rr]);
            store_frag<F>(A.out1, A.out_dtype, off[rr], valid, a[rr]);
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
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            load_frag<F>(A.in0, A.in_dtype, off[rr], valid, y[rr]);
            load_frag<F>(A.in1, A.in_dtype, off[rr], valid, b[rr]);
        }
        inverse_steps<NC, EC, R, F, TANH_ONLY, INDEXED>(y, b, wi, wj, A.tab, lane, slots, live);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            store_frag<F>(A.out0, A.out_dtype, off[rr], valid, y[rr]);
            store_frag<F>(A.out1, A.out_dtype, off[rr], valid, b[rr]);
        }
    }
}

// Tiles of up to 16 elements per lane fit 128 VGPRs (4 waves per SIMD) when the compiler is asked to; measured 3-4 %
// faster than the 136 it picks by itself.  Larger tiles, the multi-activation build and the builds that mask steps
// would spill, so they are left alone.
template <int NC, int EC, int R, int F, bool TANH_ONLY = true, bool INDEXED = false>
__global__ void __launch_bounds__(kBlockThreads, (TANH_ONLY && R * F <= 16 && F == 4) ? 4 : 1) stage_backward_kernel(const StageArgs A) {
    NCN_WAVE_PROLOGUE
    float dwi[F], dwj[F];
#pragma unroll
    for (int f = 0; f < F; ++f) dwi[f] = dwj[f] = 0.f;

    for (uint32_t t = gwave / A.n_head; t < A.total_tiles; t += tile_step) {
        int64_t off[R];
        const int live = tile_offsets<NC, EC, R, F, INDEXED>(A, t, lane, head, off);
        float Y[R][F], B[R][F], G[R][F], H[R][F];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const bool valid = INDEXED ? NCN_ROW_LIVE(rr) : live != 0;
            load_frag<F>(A.in0, A.in_dtype, off[rr], valid, Y[rr]);
            load_frag<F>(A.in1, A.in_dtype, off[rr], valid, B[rr]);
            load_frag<F>(A.g0, A.g_dtype, off[rr], valid, G[rr]);
            load_frag<F>(A.g1, A.g_dtype, off[rr], valid && A.g1 != nullptr, H[rr]);
        }
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
                    Y[rr][f] *= A.tab.inv_m_pow_n;
                    B[rr][f] *= A.tab.inv_m_pow_n;
                }
                store_frag<F>(A.aux0, NCN_F32, off[rr], valid, Y[rr]);
                store_frag<F>(A.aux1, NCN_F32, off[rr], valid, B[rr]);
            }
        }
    }

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
#undef NCN_WAVE_PROLOGUE

}  // namespace ncn
