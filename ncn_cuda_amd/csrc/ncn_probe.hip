// A measurement aid, not part of the layer: kernels that do nothing but issue one kind of vector instruction (or a mix
// shaped like the step code of the NCN kernels), so that a benchmark can quote what this GPU sustains next to what the
// NCN kernels reach.  The library is built without packed FP32 instructions; these kernels are built the same way.
// What they measured on gfx950: profiles/ has the table; in short, a vector instruction with vector-register sources
// issues once per 2.4-2.7 cycles per SIMD, one of a run of instructions that all read scalar registers, or one with a DPP
// operand, once per 4-5, v_exp_f32 / v_rcp_f32 once per 8-10, and none of these hides behind another.
//
// A launch is `waves_per_simd` workgroups of 256 threads per CU (one wave per SIMD each); the dynamic LDS a workgroup
// asks for keeps a CU from taking more.  Every lane runs `chains` independent dependency chains for
// iters x 8 "groups" of instructions each; ncn_probe_issue_info() says how many vector instructions and floating-point
// operations a group counts.  Timed by the caller (events on the stream).
#include <hip/hip_runtime.h>

#include "../../include/ncn_hip.h"

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kUnroll = 8;   // groups per chain and loop trip

// Operand forms are fixed with inline assembly where they matter: a vector instruction whose sources are all vector
// registers (or inline constants) issues about twice as often as a stream of instructions that each read a scalar
// register, and the compiler would keep the wave-uniform operands of a benchmark loop in scalar registers.
__device__ __forceinline__ float held_in_vgpr(float s) {
    float v = s;
    asm volatile("" : "+v"(v));
    return v;
}

template <int MODE, int CHAINS>
__global__ void __launch_bounds__(256) issue_kernel(float* out, int iters, float b, float c) {
    extern __shared__ float probe_lds[];
    float a[CHAINS], x[CHAINS], y[CHAINS];
#pragma unroll
    for (int k = 0; k < CHAINS; ++k) {
        a[k] = b + threadIdx.x * 1e-3f + k;
        x[k] = held_in_vgpr(1.0f + (k + 1) * 1e-7f);
        y[k] = held_in_vgpr(c * 1e-6f * (k + 1));
    }
    const float vb = held_in_vgpr(b), vc = held_in_vgpr(c);
    f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
            for (int k = 0; k < CHAINS; ++k) {
                const int nth = u * CHAINS + k;   // position in the loop body
                if (MODE == NCN_PROBE_FMA) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(x[k]), "v"(y[k]));
                if (MODE == NCN_PROBE_ADD) asm volatile("v_add_f32_e32 %0, %1, %0" : "+v"(a[k]) : "v"(y[k]));
                if (MODE == NCN_PROBE_MUL) asm volatile("v_mul_f32_e32 %0, %1, %0" : "+v"(a[k]) : "v"(x[k]));
                if (MODE == NCN_PROBE_EXP2) a[k] = __builtin_amdgcn_exp2f(a[k]);
                if (MODE == NCN_PROBE_RCP) a[k] = __builtin_amdgcn_rcpf(a[k]);
                if (MODE == NCN_PROBE_EXP2_ADD_RCP) a[k] = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(a[k]) + 1.0f);
                if (MODE == NCN_PROBE_DPP_ADD)   // v_add_f32 with a quad_perm operand: the sums across 2 and 4 lanes
                    a[k] += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(a[k]), 0xB1, 0xF, 0xF, true));
                if (MODE == NCN_PROBE_SWIZZLE_ADD)   // ds_swizzle (LDS crossbar, no memory) + v_add_f32: across 8 lanes and more
                    a[k] += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(a[k]), (4 << 10) | 0x1F));
                if (MODE == NCN_PROBE_BACKWARD_MIX) {   // 13 fma, 4 add (two of them across lanes), 1 mul, exp2, rcp
                    const float z = fmaf(a[k], vb, vc);
                    const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
                    const float w = fmaf(-r, r, r);
                    const float U = a[k] * w;
                    float g = fmaf(U, vb, vc);
                    g = fmaf(g, vb, U); g = fmaf(g, vc, r); g = fmaf(g, vb, w); g = fmaf(g, vc, z); g = fmaf(g, vb, vc);
                    g = fmaf(g, vc, vb); g = fmaf(g, vb, U); g = fmaf(g, vc, r); g = fmaf(g, vb, vc); g = fmaf(g, vc, w);
                    g += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(g), 0xB1, 0xF, 0xF, true));
                    g += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(g), (4 << 10) | 0x1F));
                    a[k] = g + vc;
                }
                if (MODE == NCN_PROBE_FORWARD_MIX) {   // 5 fma, 2 add (one across lanes), exp2, rcp
                    const float z = fmaf(a[k], vb, vc);
                    const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(z) + 1.0f);
                    float g = fmaf(r, vb, fmaf(a[k], vc, vb));
                    g = fmaf(g, vb, z); g = fmaf(g, vc, r);
                    g += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(g), 0xB1, 0xF, 0xF, true));
                    a[k] = g;
                }
                if (MODE == NCN_PROBE_MFMA) {   // v_mfma_f32_16x16x4_f32, one per chain in turn (one accumulator, reused)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[k], vb, acc, 0, 0, 0);
                }
                if (MODE == NCN_PROBE_FMA_AND_MFMA) {   // 4 fma, then one matrix instruction that depends on none of them
                    asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(x[k]), "v"(y[k]));
                    asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(y[k]), "v"(x[k]));
                    asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(x[k]), "v"(y[k]));
                    asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(y[k]), "v"(x[k]));
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(vb, vc, acc, 0, 0, 0);
                }
                if (MODE == NCN_PROBE_FMA_SGPR) asm volatile("v_fmac_f32_e32 %0, %1, %2" : "+v"(a[k]) : "s"(c), "v"(y[k]));
                if (MODE == NCN_PROBE_FMA_SGPR_1_IN_4) {
                    if (nth % 4 == 0) asm volatile("v_fmac_f32_e32 %0, %1, %2" : "+v"(a[k]) : "s"(c), "v"(y[k]));
                    else asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(x[k]), "v"(y[k]));
                }
                if (MODE == NCN_PROBE_EXP2_1_IN_8) {
                    if (nth % 8 == 0) a[k] = __builtin_amdgcn_exp2f(a[k]);
                    else asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(x[k]), "v"(y[k]));
                }
                if (MODE == NCN_PROBE_DPP_1_IN_2) {
                    if (nth % 2 == 0) a[k] += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(a[k]), 0xB1, 0xF, 0xF, true));
                    else asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[k]) : "v"(x[k]), "v"(y[k]));
                }
            }
        }
    }
    float s = acc[0] + acc[1] + acc[2] + acc[3];
#pragma unroll
    for (int k = 0; k < CHAINS; ++k) s += a[k];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s + probe_lds[0] * 0.f;
}

template <int MODE>
hipError_t launch(int chains, int blocks, size_t lds, int iters, float* out, hipStream_t s) {
    auto go = [&](auto kernel) -> hipError_t {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), lds, s, out, iters, 1.0001f, 0.25f);
        return hipGetLastError();
    };
    if (chains == 1) return go(issue_kernel<MODE, 1>);
    if (chains == 4) return go(issue_kernel<MODE, 4>);
    return go(issue_kernel<MODE, 8>);
}

}  // namespace

extern "C" int ncn_probe_issue_info(int mode, int* valu_per_group, int* flops_per_group) {
    // the mixes of one instruction in 2 and 8 with FMAs report no operation count (0): only their time per instruction means something
    static const int valu[NCN_PROBE_MODES] = {1, 1, 1, 1, 1, 3, 1, 1, 20, 9, 1, 5, 1, 1, 1, 1};
    static const int flops[NCN_PROBE_MODES] = {2, 1, 1, 1, 1, 3, 1, 1, 28, 13, 2048 / 64, 8 + 2048 / 64, 2, 2, 0, 0};
    if (mode < 0 || mode >= NCN_PROBE_MODES) return NCN_ERR_SHAPE;
    if (valu_per_group) *valu_per_group = valu[mode];
    if (flops_per_group) *flops_per_group = flops[mode];
    return kUnroll;   // groups per chain and unit of `iters`
}

extern "C" int ncn_probe_issue(int mode, int chains, int waves_per_simd, int iters, float* out, void* stream) {
    if (!out) return NCN_ERR_NULL;
    if (mode < 0 || mode >= NCN_PROBE_MODES || (chains != 1 && chains != 4 && chains != 8) || iters < 1) return NCN_ERR_SHAPE;
    if (waves_per_simd != 1 && waves_per_simd != 2 && waves_per_simd != 4 && waves_per_simd != 8) return NCN_ERR_SHAPE;
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return (int)err;
    int cus = 0;
    err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess) return (int)err;
    const int blocks = cus * waves_per_simd;                    // `out` holds blocks * 256 floats: at most 8 * CUs * 256
    const size_t lds = (160 * 1024) / waves_per_simd - (waves_per_simd == 1 ? 0 : 512);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (mode) {
        case NCN_PROBE_FMA: err = launch<NCN_PROBE_FMA>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_ADD: err = launch<NCN_PROBE_ADD>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_MUL: err = launch<NCN_PROBE_MUL>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_EXP2: err = launch<NCN_PROBE_EXP2>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_RCP: err = launch<NCN_PROBE_RCP>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_EXP2_ADD_RCP: err = launch<NCN_PROBE_EXP2_ADD_RCP>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_DPP_ADD: err = launch<NCN_PROBE_DPP_ADD>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_SWIZZLE_ADD: err = launch<NCN_PROBE_SWIZZLE_ADD>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_BACKWARD_MIX: err = launch<NCN_PROBE_BACKWARD_MIX>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_FORWARD_MIX: err = launch<NCN_PROBE_FORWARD_MIX>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_MFMA: err = launch<NCN_PROBE_MFMA>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_FMA_AND_MFMA: err = launch<NCN_PROBE_FMA_AND_MFMA>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_FMA_SGPR: err = launch<NCN_PROBE_FMA_SGPR>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_FMA_SGPR_1_IN_4: err = launch<NCN_PROBE_FMA_SGPR_1_IN_4>(chains, blocks, lds, iters, out, s); break;
        case NCN_PROBE_EXP2_1_IN_8: err = launch<NCN_PROBE_EXP2_1_IN_8>(chains, blocks, lds, iters, out, s); break;
        default: err = launch<NCN_PROBE_DPP_1_IN_2>(chains, blocks, lds, iters, out, s); break;
    }
    return (int)err;
}
