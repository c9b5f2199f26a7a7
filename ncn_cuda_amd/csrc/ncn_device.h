// Device-side building blocks shared by the NCN stage kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ncn_hip.h"

namespace ncn {

// Scalars of the recurrence, made on the host in double precision and read by the kernels through scalar loads.
//
// The register kernels do not carry x and xa themselves but
//     xs = kappa x,   as = kappa (1-m) xa          (forward)
//     xs = kappa x,   bh = kappa (1-m)/m xa        (inverse and backward),
// with kappa = 2 log2(e) alpha, and weights scaled by gamma = (1-alpha) / (2 log2(e) alpha^2).  Then
//     z = 2 log2(e) T = xs_i + c_i xs_j,   c_i = <xs_i, gamma Wi> + <xs_j, gamma Wj>       (one FMA per element),
//     forward:  as' = m as + k2 F,          xs' = m xs + as'                 (k2 = kappa (1-m)^2)
//     inverse:  xs = xs'/m - bh',           bh = bh'/m - (k2/m^2) F
// and with F = tanh T = 1 - 2r, r = 1/(1 + 2^z), the constant parts fold into the FMAs.
// The backward carries its gradients divided by m^t after t inversion steps (G = g/m^t, P = p/m^t, p = (1-m) g + h),
// which turns g <- m g + .. and p <- (1-m) g + m p into one FMA each; only dW needs the true scale, krho[t].
// The scaling needs alpha and 1-m away from zero: the host sends other values to the generic kernels.
struct StepTable {
    float alpha, m;
    int32_t activation;          // activation code (only read by kernels built for more than tanh)
    int32_t reserved;
    float kappa, inv_kappa;      // 2 log2(e) alpha
    float a_scale, inv_a_scale;  // kappa (1-m): xa -> as
    float b_scale, inv_b_scale;  // kappa (1-m)/m: xa -> bh
    float gamma;                 // (1-alpha) / (2 log2(e) alpha^2)
    float om, im;                // 1-m, 1/m
    float k2, m2k2;              // kappa (1-m)^2 and -2 k2
    float bk0, bk1;              // -k2/m^2 and 2 k2/m^2
    float ku;                    // 4 (1-m) alpha / m:  G += ku (U + rho Wi'),  U = P F'/4
    float m_pow_n, inv_m_pow_n;  // m^n_cache and its reciprocal
    float reserved2;
    float krho[64];              // (1-alpha) 4 (1-m) m^t / kappa^2: dW scale after t inversion steps
};

// Everything one stage launch needs.  Which pointer means what depends on the kernel:
//   forward : in0,in1 = x,xa        out0,out1 = y,ya      aux0,aux1 = optional float32 copies of y,ya
//   inverse : in0,in1 = y,ya        out0,out1 = x,xa
//   backward: in0,in1 = y,ya        g0,g1 = dy,dya (g1 may be null = zeros)
//             out0,out1 = dx,dxa    aux0,aux1 = optional float32 reconstructed x,xa
// Grouping: slot o of group g sits at position table[g * n_cache + o] when a table is given, at the radix-n digit
// position (g div s) * n * s + o * s + g mod s when radix_stride = s is set, else at the stride permutation's
// ((g + o * stride) % groups) * n_cache + o.  With ctx_len, batch entry b only has its first
// ctx_len[b] slots (in group order); the launches split the work: `edge == 0` runs the groups that are wholly
// live, `edge == 1` (generic kernel only) the one partly live group of each batch entry.
struct StageArgs {
    const void* in0;
    const void* in1;
    const void* g0;
    const void* g1;
    void* out0;
    void* out1;
    float* aux0;
    float* aux1;
    const float* W;      // [2E] of this stage
    float* dw_partials;  // backward: [partial rows][2E]
    const int32_t* table;    // [N] slot -> position, or null
    const int32_t* ctx_len;  // [batch] live slots per batch entry, or null
    int64_t N, E;
    int64_t plane;            // batch * N * E: elements between the two planes of an NCN_BF16X2 buffer
    uint32_t total_tiles;     // batch * tiles_per_instance
    uint32_t tiles_per_inst;  // ceil(groups / groups-per-wave-tile)
    uint32_t groups;          // N / n_cache
    uint32_t stride;          // stride of this stage in blocks: 0, or 2^(stage-1) mod groups
    uint32_t groups_pow2;     // 1 when `groups` is a power of two
    int32_t n_cache, head_dim, n_head;
    int32_t in_dtype, g_dtype, out_dtype;
    int32_t activation;
    int32_t edge;
    uint32_t radix_stride;   // n_cache^level: groups are the radix-n digit groups of that level (0: not used)
    uint32_t reserved;
    StepTable tab;
};

// ---------------------------------------------------------------------------------------------
// bfloat16 <-> float32 (round to nearest even; NaN stays NaN)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// two floats -> packed bf16 pair (lo in bits 0..15): one v_cvt_pk_bf16_f32 on gfx950, round to nearest even
typedef __bf16 ncn_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ncn_floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const ncn_floatx2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, ncn_bf16x2));
}

// Row fragment of FPL consecutive features, element offset `off` into a buffer of type `dtype`.
// NCN_BF16X2: the value is the sum of the two planes, `plane` elements apart.
template <int FPL>
__device__ __forceinline__ void load_frag(const void* base, int dtype, int64_t off, bool valid, float (&v)[FPL],
                                          int64_t plane = 0) {
    static_assert(FPL % 4 == 0, "fragment must be a multiple of 4 features");
    if (!valid) {
#pragma unroll
        for (int f = 0; f < FPL; ++f) v[f] = 0.f;
        return;
    }
    if (dtype == NCN_F32) {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(base) + off);
#pragma unroll
        for (int k = 0; k < FPL / 4; ++k) {
            float4 t = p[k];
            v[4 * k + 0] = t.x; v[4 * k + 1] = t.y; v[4 * k + 2] = t.z; v[4 * k + 3] = t.w;
        }
    } else {
        const uint2* p = reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + off);
#pragma unroll
        for (int k = 0; k < FPL / 4; ++k) {
            uint2 t = p[k];
            v[4 * k + 0] = bf16_to_f32(t.x & 0xffffu); v[4 * k + 1] = bf16_to_f32(t.x >> 16);
            v[4 * k + 2] = bf16_to_f32(t.y & 0xffffu); v[4 * k + 3] = bf16_to_f32(t.y >> 16);
        }
        if (dtype == NCN_BF16X2) {
            const uint2* q = reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + off + plane);
#pragma unroll
            for (int k = 0; k < FPL / 4; ++k) {
                uint2 t = q[k];
                v[4 * k + 0] += bf16_to_f32(t.x & 0xffffu); v[4 * k + 1] += bf16_to_f32(t.x >> 16);
                v[4 * k + 2] += bf16_to_f32(t.y & 0xffffu); v[4 * k + 3] += bf16_to_f32(t.y >> 16);
            }
        }
    }
}

template <int FPL>
__device__ __forceinline__ void store_frag(void* base, int dtype, int64_t off, bool valid, const float (&v)[FPL],
                                           int64_t plane = 0) {
    if (!valid) return;
    if (dtype == NCN_F32) {
        float4* p = reinterpret_cast<float4*>(static_cast<float*>(base) + off);
#pragma unroll
        for (int k = 0; k < FPL / 4; ++k) p[k] = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
    } else {
        uint2* p = reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + off);
#pragma unroll
        for (int k = 0; k < FPL / 4; ++k) {
            uint2 t;
            t.x = pack_bf16x2(v[4 * k + 0], v[4 * k + 1]);
            t.y = pack_bf16x2(v[4 * k + 2], v[4 * k + 3]);
            p[k] = t;
            if (dtype == NCN_BF16X2) {   // second plane: what the rounding took away (the difference is exact in float32)
                uint2 u;
                u.x = pack_bf16x2(v[4 * k + 0] - bf16_to_f32(t.x & 0xffffu), v[4 * k + 1] - bf16_to_f32(t.x >> 16));
                u.y = pack_bf16x2(v[4 * k + 2] - bf16_to_f32(t.y & 0xffffu), v[4 * k + 3] - bf16_to_f32(t.y >> 16));
                reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + off + plane)[k] = u;
            }
        }
    }
}

// A register tile on its way from global memory: R row fragments of FPL features, still as loaded.  issue() only
// requests the data (one branch on the element type around all the loads of the tile), finish() turns it into floats:
// a kernel issues the loads of all its input tiles before it finishes the first, so that their latencies overlap
// instead of following one another (converting each fragment as it is loaded waits for every load in turn).
// The offsets must be valid addresses for every lane (lanes without work read some row of their own batch entry and
// are zeroed afterwards where that matters).
template <int R, int FPL>
__device__ __forceinline__ void issue_tile(const void* base, int dtype, const int64_t (&off)[R], float (&v)[R][FPL],
                                           int64_t plane = 0) {
    static_assert(FPL % 4 == 0, "fragment must be a multiple of 4 features");
    // the registers of the fragment hold the raw words until finish_tile: float32 all four of a chunk, bfloat16 the
    // first two, two planes the value plane in the first two and the residual plane in the last two
    if (dtype == NCN_F32) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int k = 0; k < FPL / 4; ++k) {
                const float4 t = reinterpret_cast<const float4*>(static_cast<const float*>(base) + off[rr])[k];
                v[rr][4 * k] = t.x; v[rr][4 * k + 1] = t.y; v[rr][4 * k + 2] = t.z; v[rr][4 * k + 3] = t.w;
            }
    } else if (dtype == NCN_BF16) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int k = 0; k < FPL / 4; ++k) {
                const float2 t = reinterpret_cast<const float2*>(static_cast<const uint16_t*>(base) + off[rr])[k];
                v[rr][4 * k] = t.x; v[rr][4 * k + 1] = t.y;
            }
    } else {
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int k = 0; k < FPL / 4; ++k) {
                const float2 t = reinterpret_cast<const float2*>(static_cast<const uint16_t*>(base) + off[rr])[k];
                const float2 u = reinterpret_cast<const float2*>(static_cast<const uint16_t*>(base) + off[rr] + plane)[k];
                v[rr][4 * k] = t.x; v[rr][4 * k + 1] = t.y; v[rr][4 * k + 2] = u.x; v[rr][4 * k + 3] = u.y;
            }
    }
}

template <int R, int FPL>
__device__ __forceinline__ void finish_tile(int dtype, float (&v)[R][FPL]) {
    if (dtype == NCN_F32) return;
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
        for (int k = 0; k < FPL / 4; ++k) {
            float* o = &v[rr][4 * k];
            const uint32_t w0 = __float_as_uint(o[0]), w1 = __float_as_uint(o[1]);
            const uint32_t r0 = __float_as_uint(o[2]), r1 = __float_as_uint(o[3]);
            o[0] = __uint_as_float(w0 << 16); o[1] = __uint_as_float(w0 & 0xffff0000u);
            o[2] = __uint_as_float(w1 << 16); o[3] = __uint_as_float(w1 & 0xffff0000u);
            if (dtype == NCN_BF16X2) {
                o[0] += __uint_as_float(r0 << 16); o[1] += __uint_as_float(r0 & 0xffff0000u);
                o[2] += __uint_as_float(r1 << 16); o[3] += __uint_as_float(r1 & 0xffff0000u);
            }
        }
}

__device__ __forceinline__ float load_elem(const void* base, int dtype, int64_t off, int64_t plane = 0) {
    if (dtype == NCN_F32) return static_cast<const float*>(base)[off];
    const uint16_t* p = static_cast<const uint16_t*>(base);
    return dtype == NCN_BF16X2 ? bf16_to_f32(p[off]) + bf16_to_f32(p[off + plane]) : bf16_to_f32(p[off]);
}

__device__ __forceinline__ void store_elem(void* base, int dtype, int64_t off, float v, int64_t plane = 0) {
    if (dtype == NCN_F32) {
        static_cast<float*>(base)[off] = v;
    } else {
        uint16_t* p = static_cast<uint16_t*>(base);
        const uint32_t hi = f32_to_bf16(v);
        p[off] = static_cast<uint16_t>(hi);
        if (dtype == NCN_BF16X2) p[off + plane] = static_cast<uint16_t>(f32_to_bf16(v - bf16_to_f32(hi)));
    }
}

// ---------------------------------------------------------------------------------------------
// cross-lane moves inside one 64-wide wavefront
// ---------------------------------------------------------------------------------------------
// value of lane (lane ^ S).  ROWS: stride 8 as a DPP row rotation instead of a trip through the LDS crossbar
// (costs the same issue slots, and on kernels that are bound by issue a little more through its wait states; pays
// on kernels that wait on latency).
template <int S, bool ROWS = false>
__device__ __forceinline__ float lane_xor(float v) {
    static_assert(S == 1 || S == 2 || S == 4 || S == 8 || S == 16 || S == 32, "power of two below 64");
    int x = __float_as_int(v);
    if constexpr (S == 1) {
        x = __builtin_amdgcn_mov_dpp(x, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
    } else if constexpr (S == 2) {
        x = __builtin_amdgcn_mov_dpp(x, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
    } else if constexpr (S == 8 && ROWS) {
        x = __builtin_amdgcn_update_dpp(0, x, 0x128, 0xF, 0xF, true);  // row_ror:8 == lane ^ 8 inside a row of 16
    } else if constexpr (S < 32) {
        x = __builtin_amdgcn_ds_swizzle(x, (S << 10) | 0x1F);   // bit mode: lane' = lane ^ S inside 32
    } else {
        const int lane = __lane_id();
        x = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, x);
    }
    return __int_as_float(x);
}

// sum over the lanes {lane ^ k*LO : k} for strides LO, 2*LO, .. < HI  (LO, HI powers of two).
// ROWS (see lane_xor): when the recursion started at stride 1 (FROM1), the value is the same in the four lanes of a
// quad from stride 4 on, and the partner quad is read through row_half_mirror (lane 7 - i of each 8).
template <int LO, int HI, bool ROWS = false, bool FROM1 = (LO == 1)>
__device__ __forceinline__ float lane_sum(float v) {
    if constexpr (LO < HI) {
        if constexpr (LO == 4 && FROM1 && ROWS)
            v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
        else
            v += lane_xor<LO, ROWS>(v);
        return lane_sum<LO * 2, HI, ROWS, FROM1>(v);
    } else {
        return v;
    }
}

// The same sums for N values at once, level by level over all of them: the N chains are independent, so their trips
// across the lanes overlap (one wait per level instead of one per value and level).
template <int LO, int HI, bool ROWS, int N, bool FROM1 = (LO == 1)>
__device__ __forceinline__ void lane_sum_n(float (&v)[N]) {
    if constexpr (LO < HI) {
#pragma unroll
        for (int k = 0; k < N; ++k) {
            if constexpr (LO == 4 && FROM1 && ROWS)
                v[k] += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v[k]), 0x141, 0xF, 0xF, true));
            else
                v[k] += lane_xor<LO, ROWS>(v[k]);
        }
        lane_sum_n<LO * 2, HI, ROWS, N, FROM1>(v);
    }
}

// value held by lane `src_lane` (any lane of the wave; computed at run time).  ds_bpermute is several times
// slower than ds_swizzle/DPP on gfx950: keep it off hot paths.
__device__ __forceinline__ float lane_read(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}

// Lane bits [log2(LF), log2(LF*LR)) hold a "row lane" index; every lane receives the F-register fragment of the
// lane that has the same other bits and row lane index `jo` (uniform, known only at run time).
// Through LDS: every lane stores its fragment into its own slot of a wave-private buffer and loads the slot of
// its source lane (one ds_write + one ds_read of 16 bytes per 4 registers; a wave's LDS operations complete in
// issue order, so no barrier is needed).  ds_bpermute would do the same without memory but costs about six
// times an FMA per register on gfx950, and a switch over ds_swizzle patterns wrecks register allocation.
template <int LF, int LR, int F>
__device__ __forceinline__ void row_lane_broadcast(const float (&v)[F], float (&out)[F], int jo, int lane,
                                                   float4* wave_slots) {
    if constexpr (LR == 1) {
#pragma unroll
        for (int f = 0; f < F; ++f) out[f] = v[f];
    } else {
        static_assert(F % 4 == 0, "fragments are stored as float4");
        const int src = (lane & ~((LR - 1) * LF)) | (jo * LF);
#pragma unroll
        for (int k = 0; k < F / 4; ++k) wave_slots[k * 64 + lane] = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
#pragma unroll
        for (int k = 0; k < F / 4; ++k) {
            const float4 t = wave_slots[k * 64 + src];
            out[4 * k] = t.x; out[4 * k + 1] = t.y; out[4 * k + 2] = t.z; out[4 * k + 3] = t.w;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// activation: F(T) and dF/dT.  Codes of the reference's CUDA kernels
// (ncn_fwd_cuda_kernel.cu:86-95, ncn_bwd_cuda_kernel.cu:137-150).
// ---------------------------------------------------------------------------------------------
// tanh(T) = 1 - 2/(1 + e^{2T}) with the hardware exp2 and reciprocal (about 1 ulp each): the absolute
// error of F stays near 1e-7 over the whole range, and the saturated ends come out exactly +-1.
__device__ __forceinline__ void tanh_fd(float T, float& F, float& dF) {
    const float t = __builtin_amdgcn_exp2f(T * 2.8853900817779268f);
    const float r = __builtin_amdgcn_rcpf(t + 1.0f);
    F = fmaf(-2.0f, r, 1.0f);
    dF = 4.0f * r * (1.0f - r);  // 1 - F^2
}

__device__ __forceinline__ float tanh_f(float T) {
    const float t = __builtin_amdgcn_exp2f(T * 2.8853900817779268f);
    const float r = __builtin_amdgcn_rcpf(t + 1.0f);
    return fmaf(-2.0f, r, 1.0f);
}

__device__ __forceinline__ void act_fd(int code, float T, float& F, float& dF) {
    if (code == NCN_ACT_TANH) {
        tanh_fd(T, F, dF);
    } else if (code == NCN_ACT_RELU) {
        F = fmaxf(T, 0.f);
        dF = F > 0.f ? 1.f : 0.f;
    } else if (code == NCN_ACT_SIGMOID) {
        const float t = __builtin_amdgcn_exp2f(-T * 1.4426950408889634f);
        F = __builtin_amdgcn_rcpf(1.0f + t);
        dF = F * (1.0f - F);
    } else if (code == NCN_ACT_LEAKY_RELU) {
        F = T >= 0.f ? T : 0.01f * T;
        dF = T >= 0.f ? 1.f : 0.01f;
    } else {
        F = T;
        dF = 1.f;
    }
}

// ---------------------------------------------------------------------------------------------
// stride permutation (torch_ref/ncn_pytorch.py:38-40): block that slot `slot` of group `group` reads
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t stage_block(const StageArgs& A, uint32_t group, uint32_t slot) {
    const uint32_t t = group + slot * A.stride;  // < 65 * groups, checked on the host to fit 32 bits
    return A.groups_pow2 ? (t & (A.groups - 1u)) : (t % A.groups);
}

// Position on the N axis of slot `slot` of group `group`.  A table entry is clamped into [0, N): a table that is
// not a permutation gives wrong numbers, never an access outside the tensors.
__device__ __forceinline__ int64_t slot_position(const StageArgs& A, uint32_t group, uint32_t slot) {
    if (A.table) {
        const int32_t p = A.table[(int64_t)group * A.n_cache + slot];
        return (int64_t)max(0, min(p, (int32_t)A.N - 1));
    }
    if (A.radix_stride) {   // the positions that differ only in one base-n digit (ncn_triton/group_tensors.py:8-18)
        const uint32_t s = A.radix_stride, hi = group / s;
        return ((int64_t)hi * A.n_cache + slot) * s + (group - hi * s);
    }
    return (int64_t)stage_block(A, group, slot) * A.n_cache + slot;
}

// Live slots of batch entry b (ncn_triton/ncn_triton_old.py:66: one context length per batch entry).
__device__ __forceinline__ int32_t live_slots(const StageArgs& A, uint32_t b) {
    return A.ctx_len ? max(0, min(A.ctx_len[b], (int32_t)A.N)) : (int32_t)A.N;
}

// Live rows of group `group` of batch entry b: n_cache, fewer for the group the length cuts, 0 beyond it.
__device__ __forceinline__ int32_t live_rows(const StageArgs& A, uint32_t b, uint32_t group) {
    if (!A.ctx_len) return A.n_cache;
    const int64_t r = (int64_t)live_slots(A, b) - (int64_t)group * A.n_cache;
    return (int32_t)max((int64_t)0, min(r, (int64_t)A.n_cache));
}

}  // namespace ncn
