/*
 * ncn_hip.h -- C ABI of the MI355X (gfx950) NCN layer library, libncn_hip.so.
 *
 * The library replaces the reference's pybind11 module `ncn_cuda_module`
 * (ncn_cuda/ncn_cuda.cpp:29-32, built from ncn_fwd_cuda_kernel.cu and ncn_bwd_cuda_kernel.cu).
 * Differences of contract with that module, all deliberate:
 *   - the caller owns every buffer (inputs, outputs, workspace); the library never allocates,
 *     frees or keeps a pointer after a call returns        (reference: torch::zeros_like inside,
 *     ncn_fwd_cuda_kernel.cu:128-129, ncn_bwd_cuda_kernel.cu:247-251);
 *   - work is enqueued on the HIP stream passed in and the call returns without a host sync
 *     (reference: default stream + cudaDeviceSynchronize, ncn_fwd_cuda_kernel.cu:158);
 *   - every entry point returns 0 or an error code (reference: no checks at all);
 *   - activations and gradients may be float32 or bfloat16 in memory; all arithmetic is float32;
 *     W and dW are always float32;
 *   - `m`, hard-coded to 0.9 in the reference (ncn_fwd_cuda_kernel.cu:72), is an argument;
 *   - several consecutive stages can be run by one call (n_stages > 1), later stages in place.
 *
 * Tensors are row-major [batch, N, E] with E contiguous; a head is a slice of E/n_head features.
 * Stage `l` of the layer groups the N axis into N/n_cache groups of n_cache rows through the
 * stride permutation of torch_ref/ncn_pytorch.py:12-41 and runs the n_cache-step recurrence of
 * torch_ref/ncn_pytorch.py:74-94 on each (batch, head, group).  W holds, per stage, 2E floats:
 * W[0:E] multiplies the row itself (Wi), W[E:2E] the step's pivot row (Wj); a head uses its own
 * slice of both halves (torch_ref/ncn_pytorch.py:60-61).
 *
 * All pointers are device pointers, 16-byte aligned.  Calls are re-entrant; two calls that write the
 * same buffers must be ordered by the caller (same stream, or events).  Kernels are launched on `stream`
 * (NULL: the default stream) of the device that is current when the call is made: make the device that
 * owns the buffers and the stream current first (hipSetDevice).
 */
#ifndef NCN_HIP_H
#define NCN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of activation / gradient buffers */
#define NCN_F32 0
#define NCN_BF16 1
/* A value kept as two bfloat16: buffer [2, batch, N, E], plane 0 = the value rounded to bfloat16, plane 1 = what
 * the rounding took away, rounded to bfloat16 again (16 significant bits in all).  What a bf16 caller saves for the
 * reversible backward: plane 0 alone is the ordinary bf16 tensor [batch, N, E] (the next stage reads it as NCN_BF16),
 * so a forward writes 4 bytes per value instead of the 2 + 4 of a bf16 output plus a float32 copy.  Accepted as
 * out_dtype of ncn_forward / ncn_forward_indexed, y_dtype of ncn_backward / ncn_backward_indexed / ncn_backward_static
 * and in_dtype of ncn_inverse / ncn_inverse_indexed, for one stage per call (n_stages == 1) on the register kernels
 * (ncn_kernel_path() == 2); NCN_ERR_DTYPE elsewhere. */
#define NCN_BF16X2 2

/* activation codes: those of the reference's CUDA surface (ncn_pytorch_wrapper_v2.py:111,
 * ncn_fwd_cuda_kernel.cu:86-95): 0 tanh, 1 relu, 2 sigmoid, anything else the reference treats as
 * linear; here only -1 is accepted for linear.  Code 3 is the leaky relu of the reference's Triton kernels
 * (ncn_triton/ncn_triton.py:22-28, 101-102: slope 0.01 below zero, value and slope of the upper branch at 0),
 * which the CUDA surface does not have. */
#define NCN_ACT_TANH 0
#define NCN_ACT_RELU 1
#define NCN_ACT_SIGMOID 2
#define NCN_ACT_LEAKY_RELU 3
#define NCN_ACT_LINEAR (-1)

/* error codes (negative: rejected before any GPU work; positive: a hipError_t from the runtime) */
#define NCN_OK 0
#define NCN_ERR_NULL (-1)        /* a required pointer is NULL */
#define NCN_ERR_SHAPE (-2)       /* non-positive size, N % n_cache != 0, E % n_head != 0, bad stage range */
#define NCN_ERR_DTYPE (-3)       /* unknown element type */
#define NCN_ERR_ACTIVATION (-4)  /* unknown activation code */
#define NCN_ERR_WORKSPACE (-5)   /* workspace missing or smaller than ncn_workspace_bytes() */
#define NCN_ERR_UNSUPPORTED (-6) /* n_cache > 64, or head width too large for the generic kernel; also alpha outside
                                    [1e-3, 1e3] or m outside [1e-3, 0.999] at head widths above 64 (see ncn_kernel_path_scalars) */
#define NCN_ERR_ALIGN (-7)       /* a pointer is not 16-byte aligned (4-byte for the int32 tables) */
#define NCN_ERR_ALIAS (-8)       /* n_stages > 1 needs the state buffers the call would carry it in */
#define NCN_ERR_STATIC_LIMIT (-9) /* ncn_backward_static: the shape needs more scratch than the library holds */

/* Shape of one problem; shared by all entry points. */
typedef struct ncn_shape {
    int64_t batch;   /* X.size(0) */
    int64_t N;       /* X.size(1), the mixing axis (reference: ctx_dim) */
    int64_t E;       /* X.size(2) (reference: embed_dim) */
    int32_t n_head;  /* heads; head width Ec = E / n_head (reference: nhead) */
    int32_t n_cache; /* group size (reference: cache_dim) */
} ncn_shape;

/*
 * Forward of stages first_stage .. first_stage+n_stages-1.
 * Replaces: forward(X, Xa, W, alpha, activation, cache_dim, nhead, module_l) -> {Y, Ya}
 *           ncn_cuda/ncn_cuda.cpp:3-12, ncn_fwd_cuda_kernel.cu:115-161 (one stage per call there).
 * x, xa       in   [batch,N,E] of in_dtype
 * y, ya       out  [batch,N,E] of out_dtype; may alias x, xa when the dtypes are equal (each row is
 *                  read and written by exactly one wavefront).  With n_stages > 1 the later stages
 *                  run in place on y, ya.
 * y32, ya32   out  optional (NULL to skip) float32 copies of the final y, ya: what a bf16 caller saves
 *                  for the reversible backward.
 * W           in   [n_stages, 2E] float32
 * workspace        optional scratch (NULL, 0 to skip).  With n_stages > 1 and small groups the library keeps
 *                  tiles of rows in LDS across several stages instead of launching stage by stage; when that
 *                  takes more than one pass it needs ncn_workspace_bytes_stages(.., backward = 0) bytes here
 *                  and float32 outputs, and silently falls back to one launch per stage without them.
 */
int ncn_forward(const void* x, const void* xa, int in_dtype,
                void* y, void* ya, int out_dtype,
                float* y32, float* ya32,
                const float* W,
                void* workspace, size_t workspace_bytes,
                const ncn_shape* shape, int first_stage, int n_stages,
                float alpha, float m, int activation, void* stream);

/*
 * Reversible backward of stages first_stage+n_stages-1 .. first_stage, from the OUTPUTS of the last
 * of them.
 * Replaces: backward(Y, Ya, dY, dYa, W, alpha, activation, cache_dim, nhead, module_l)
 *           -> {X, Xa, dX, dXa, dW[batch,N,2E]}  ncn_cuda/ncn_cuda.cpp:14-25,
 *           ncn_bwd_cuda_kernel.cu:232-288, plus the torch.sum(dW,(0,1)) of
 *           ncn_pytorch_wrapper_v2.py:48, which is done here.
 * y, ya       in   [batch,N,E] of y_dtype: outputs of the last stage (use float32: the inversion
 *                  amplifies rounding by (1/m)^n_cache per stage)
 * dy, dya     in   [batch,N,E] of dy_dtype; dya may be NULL, meaning zeros
 * dx, dxa     out  [batch,N,E] of dx_dtype
 * x_rec,xa_rec out float32 [batch,N,E], reconstructed inputs of first_stage, or both NULL when the caller does not
 *                  want them (an autograd node does not).  With n_stages > 1 dx_dtype must be NCN_F32 and the
 *                  four of x_rec, xa_rec, dx, dxa carry the state between stages in place; without x_rec, xa_rec
 *                  two arrays of the workspace do (ncn_workspace_bytes_stages(.., backward = 2) bytes) and the
 *                  last stage to run writes no reconstructed inputs at all (NCN_ERR_ALIAS if the workspace is
 *                  smaller).
 * W           in   [n_stages, 2E] float32
 * dW          out  [n_stages, 2E] float32, overwritten (summed over batch, groups and rows)
 * workspace        scratch of at least ncn_workspace_bytes(shape) bytes; with n_stages > 1,
 *                  ncn_workspace_bytes_stages(.., backward = 1) bytes let the library use its multi-stage
 *                  LDS-resident passes (it falls back to one launch per stage with less)
 */
int ncn_backward(const void* y, const void* ya, int y_dtype,
                 const void* dy, const void* dya, int dy_dtype,
                 void* dx, void* dxa, int dx_dtype,
                 float* x_rec, float* xa_rec,
                 const float* W, float* dW,
                 void* workspace, size_t workspace_bytes,
                 const ncn_shape* shape, int first_stage, int n_stages,
                 float alpha, float m, int activation, void* stream);

/*
 * ncn_backward without a workspace argument and without any allocation, for callers that cannot allocate device
 * memory (code under HIP graph capture, serving loops, harnesses that forbid it).  No counterpart in the reference,
 * whose host functions allocate every output and the [batch, N, 2E] dW partial tensor themselves
 * (ncn_bwd_cuda_kernel.cu:247-251).  The dW partial rows live in an array inside the library
 * (ncn_static_scratch_bytes() bytes, about 9 MiB, held by every GPU the library runs on until the process ends).
 * Limits: E <= 256 (NCN_ERR_STATIC_LIMIT above that); always one launch per stage, also where ncn_backward would use
 * its multi-stage passes, so with n_stages > 1 the two agree to rounding, not bit for bit; dx, dxa, x_rec, xa_rec of
 * one stage are bit-identical to ncn_backward's, dW sums the same terms over fewer partial rows.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (different streams or threads) race;
 * calls on one stream are ordered.  Nothing in the array has to be cleared between calls.
 * Arguments as ncn_backward, with one difference: with n_stages > 1, x_rec and xa_rec are REQUIRED (NCN_ERR_ALIAS when
 * they are NULL).  The stages of a call hand their reconstructed inputs on through them; ncn_backward takes two
 * float32 [batch, N, E] arrays from its workspace for that when they are NULL, and the library's array is far too
 * small to hold those.  With n_stages == 1 they may be NULL as there.
 * Before a stream capture: make one call of the same shape class on the device outside the capture.  The first call
 * per device resolves the array's address (hipGetSymbolAddress) and the first launch of a kernel that needs more than
 * 64 KB of LDS raises its limit (hipFuncSetAttribute); neither can be recorded into a graph.  Later calls only launch.
 */
int ncn_backward_static(const void* y, const void* ya, int y_dtype,
                        const void* dy, const void* dya, int dy_dtype,
                        void* dx, void* dxa, int dx_dtype,
                        float* x_rec, float* xa_rec,
                        const float* W, float* dW,
                        const ncn_shape* shape, int first_stage, int n_stages,
                        float alpha, float m, int activation, void* stream);

/* Size in bytes of the library's own scratch array per GPU (see ncn_backward_static). */
size_t ncn_static_scratch_bytes(void);

/*
 * Inverse of stages first_stage+n_stages-1 .. first_stage: x, xa such that ncn_forward(x, xa) = y, ya.
 * Follows NCNFunctionPytorch.invert (torch_ref/ncn_pytorch_invertible.py:87-113), which the
 * reference's CUDA module only runs inside backward (ncn_bwd_cuda_kernel.cu:88-115).
 * May run in place (x == y, xa == ya) when the dtypes are equal.  With n_stages > 1, float32 outputs and small
 * groups it uses the multi-stage LDS passes that can work without scratch (every closed pass, and a halo pass when it
 * is the first to run and x, xa are not y, ya) and one launch per stage for the rest.
 */
int ncn_inverse(const void* y, const void* ya, int in_dtype,
                void* x, void* xa, int out_dtype,
                const float* W,
                const ncn_shape* shape, int first_stage, int n_stages,
                float alpha, float m, int activation, void* stream);

/*
 * ncn_inverse with scratch: with ncn_workspace_bytes_stages(shape, first_stage, n_stages, activation, 0) bytes (the
 * forward's figure) and float32 outputs every multi-stage pass runs as one launch, halo passes included: the passes
 * read one pair of buffers and write another, scratch and x, xa in turns.  With less scratch, or where the turns would
 * make the first pass write into its own input (x == y with an odd number of passes), it does what ncn_inverse does.
 * Replaces the same reference code as ncn_inverse; the reference has no multi-stage inverse
 * (torch_ref/ncn_pytorch_invertible.py:87-113 undoes one stage per call).
 */
int ncn_inverse_ws(const void* y, const void* ya, int in_dtype,
                   void* x, void* xa, int out_dtype,
                   const float* W,
                   void* workspace, size_t workspace_bytes,
                   const ncn_shape* shape, int first_stage, int n_stages,
                   float alpha, float m, int activation, void* stream);

/*
 * The same three operations with the grouping given as a table and, optionally, one context length per batch entry.
 * Replaces: the group_tensor / ctxlen_tensor arguments of fused_chunk_linear_ncn and its kernels
 *           (ncn_triton/ncn_triton_old.py:53-57, 66-71, 93-96, 362-387), whose tables come from helpers such as the
 *           radix-n digit grouping of ncn_triton/group_tensors.py:8-18.
 * group_index in  int32 [n_stages, N], or NULL for the stride permutation of first_stage + k (first_stage is only
 *                 read then).  For stage k, slot o of group g is the row at position group_index[k*N + g*n_cache + o]
 *                 of the N axis.  Every row of the table must be a permutation of 0 .. N-1: the library cannot check
 *                 that; entries are clamped into range, so a bad table gives wrong numbers but no stray access.
 * ctx_len     in  int32 [batch], or NULL for N everywhere.  Batch entry b only has its first ctx_len[b] slots (in the
 *                 order of the table): groups wholly below the length run as usual; the group the length cuts runs
 *                 on its live rows only, with as many steps as it has live rows; rows past the length pass through
 *                 (forward, inverse: out = in; backward: dx = dy, dxa = dya, x_rec = y, no share in dW).  Values are
 *                 clamped to [0, N].
 * Everything else as in ncn_forward / ncn_backward / ncn_inverse.  With a table these run stage by stage and
 * ncn_backward_indexed needs ncn_workspace_bytes(shape) (followed, for several stages without x_rec, xa_rec, by two
 * float32 arrays of the tensors' size, each padded to a multiple of 256 bytes).  With lengths only (group_index NULL) the grouping is the
 * stride permutation and several stages use the multi-stage LDS passes where ncn_forward / ncn_inverse / ncn_backward
 * would (float32 between passes): forward and inverse take no workspace, so their first pass goes from the inputs to
 * the outputs and the others work in place on the outputs, where the stages of a halo pass run one launch each;
 * ncn_backward_indexed uses the passes when given ncn_workspace_bytes_stages(.., backward = 1) bytes.  Inside a pass
 * the rows past a length stay in LDS in the kernels' scaled form, so they come out equal to their inputs to rounding
 * (one launch per stage copies them bit for bit).
 */
int ncn_forward_indexed(const void* x, const void* xa, int in_dtype,
                        void* y, void* ya, int out_dtype,
                        float* y32, float* ya32,
                        const float* W,
                        const int32_t* group_index, const int32_t* ctx_len,
                        const ncn_shape* shape, int first_stage, int n_stages,
                        float alpha, float m, int activation, void* stream);

int ncn_backward_indexed(const void* y, const void* ya, int y_dtype,
                         const void* dy, const void* dya, int dy_dtype,
                         void* dx, void* dxa, int dx_dtype,
                         float* x_rec, float* xa_rec,
                         const float* W, float* dW,
                         void* workspace, size_t workspace_bytes,
                         const int32_t* group_index, const int32_t* ctx_len,
                         const ncn_shape* shape, int first_stage, int n_stages,
                         float alpha, float m, int activation, void* stream);

int ncn_inverse_indexed(const void* y, const void* ya, int in_dtype,
                        void* x, void* xa, int out_dtype,
                        const float* W,
                        const int32_t* group_index, const int32_t* ctx_len,
                        const ncn_shape* shape, int first_stage, int n_stages,
                        float alpha, float m, int activation, void* stream);

/*
 * Levels first_level .. first_level+n_levels-1 of the radix-n digit grouping: level l groups the n_cache positions
 * of the N axis that differ only in base-n_cache digit l (slot = that digit; the remaining digits, the upper ones
 * moved down one place, number the group).
 * Replaces: the grouping of ncn_triton/group_tensors.py:8-18 (extract_group_index), which the reference only has as a
 *           helper that writes index tensors; level 0 is stage 0 of the stride permutation.  The same levels can be
 *           run through ncn_*_indexed with tables; these entry points need no table and, for n_cache 2 or 4 with a
 *           head width of 16 or 32, keep windows of n_cache^k rows in LDS over k levels per pass (such windows are
 *           closed: no halo, every pass in place), so a stack of log_n(N) levels costs two or three passes over HBM.
 * n_cache^(first_level+n_levels) must divide N (NCN_ERR_SHAPE otherwise).  W, dW: [n_levels, 2E].
 * Arguments as in ncn_forward / ncn_backward.  Levels after the first pass run in place on y, ya (forward) and on
 * x_rec, xa_rec, dx, dxa (backward): use float32 outputs when more than one pass is needed, or the values between
 * passes are rounded to the output type.  ncn_backward_radix needs ncn_workspace_bytes(shape) of scratch; with several
 * levels x_rec, xa_rec may both be NULL when that scratch is followed by two float32 arrays of the tensors' size (each
 * padded to a multiple of 256 bytes): the last pass to run then writes no reconstructed inputs.
 */
int ncn_forward_radix(const void* x, const void* xa, int in_dtype,
                      void* y, void* ya, int out_dtype,
                      float* y32, float* ya32,
                      const float* W,
                      const ncn_shape* shape, int first_level, int n_levels,
                      float alpha, float m, int activation, void* stream);

int ncn_backward_radix(const void* y, const void* ya, int y_dtype,
                       const void* dy, const void* dya, int dy_dtype,
                       void* dx, void* dxa, int dx_dtype,
                       float* x_rec, float* xa_rec,
                       const float* W, float* dW,
                       void* workspace, size_t workspace_bytes,
                       const ncn_shape* shape, int first_level, int n_levels,
                       float alpha, float m, int activation, void* stream);

/* Inverse of ncn_forward_radix: x, xa with ncn_forward_radix(x, xa) = y, ya; may run in place. */
int ncn_inverse_radix(const void* y, const void* ya, int in_dtype,
                      void* x, void* xa, int out_dtype,
                      const float* W,
                      const ncn_shape* shape, int first_level, int n_levels,
                      float alpha, float m, int activation, void* stream);

/* How the calls above cut the levels into passes (the inverse uses the forward's cut); returns the number of passes or a negative error code and
 * writes up to max_passes records of 6 int32 into `out` (may be NULL):
 *   [0] first level of the pass relative to first_level   [1] levels in the pass   [2] 0 one-stage launch, 1 LDS windows
 *   [3] n_cache^(first level): distance in rows between the rows of a window   [4] rows of a window   [5] rows per workgroup
 * No reference counterpart. */
int ncn_plan_radix(const ncn_shape* shape, int first_level, int n_levels, int activation, int backward, int32_t* out,
                   int max_passes);

/* Bytes of scratch ncn_backward needs for this shape (0 on an invalid shape).  No reference counterpart:
 * the reference allocates a [batch,N,2E] partial-dW tensor per call (ncn_bwd_cuda_kernel.cu:251). */
size_t ncn_workspace_bytes(const ncn_shape* shape);

/* Bytes of scratch that let ncn_forward (backward = 0) or ncn_backward (backward = 1) run stages
 * first_stage .. first_stage+n_stages-1 with the multi-stage passes; never less than what the call needs anyway
 * (0 for forward, ncn_workspace_bytes for backward).  For the backward that is, in this order: a dW partial row of
 * 2E floats for every window and stage of every pass (at most 65536 rows, at least those of ncn_workspace_bytes)
 * with their chunk sums, so that every window gets a workgroup of its own, and, with two passes or more, four
 * float32 arrays of the tensors' size.  ncn_backward also takes ncn_workspace_bytes(shape) plus the four arrays
 * (each padded to a multiple of 256 bytes) and then lets its workgroups walk over several windows, which is slower.
 * backward = 2: the same for a call without x_rec, xa_rec, which takes the two arrays that carry the reconstructed
 * state between stages from the end of the workspace (none when one pass over closed rings covers the range).
 * No reference counterpart. */
size_t ncn_workspace_bytes_stages(const ncn_shape* shape, int first_stage, int n_stages, int activation, int backward);

/* How ncn_forward / ncn_backward would cut stages first_stage .. first_stage+n_stages-1 into passes, for
 * inspection and tests.  Returns the number of passes (0: one launch per stage), or a negative error code;
 * writes up to max_passes records of 8 int32 into `out` (may be NULL):
 *   [0] first stage of the pass relative to first_stage   [1] stages in the pass
 *   [2] kind: 0 one-stage launch, 1 halo window, 2 closed rings
 *   [3] class stride S0 in blocks   [4] window   [5] halo   [6] owned sub-blocks per window
 *   [7] windows per batch entry and ring tile (classes, or groups of classes for closed rings)
 * No reference counterpart. */
int ncn_plan_passes(const ncn_shape* shape, int first_stage, int n_stages, int activation, int backward, int32_t* out,
                    int max_passes);

/* 2: hand-tuned register kernel, 1: generic LDS kernel, 0: not supported (n_cache > 64, or the
 * head width does not fit the generic kernel's LDS).  Register kernels exist for n_cache 2, 4, 8, 16, 32, 64 with
 * head widths 4 .. 128 (powers of two; 128 up to n_cache 16, 64 up to 32), and for heads of one feature
 * (E == n_head, the recurrence on rows of scalars) when E is a multiple of 4: the library lays those out as heads of
 * 32, 16, 8 or 4 adjacent ones (the largest that divides E), with the multi-stage passes of such heads for n_cache 2
 * and 4 when E is a multiple of 8.  No reference counterpart. */
int ncn_kernel_path(const ncn_shape* shape);

/* The same for a call with these scalars: the register kernels carry their state times alpha and 1 - m, so values
 * of alpha or 1 - m next to zero (below 1e-3) run on the generic kernels (1), or nowhere (0) when the head is wider
 * than those take. */
int ncn_kernel_path_scalars(const ncn_shape* shape, float alpha, float m);

/* Validates the shape, stage range and activation exactly as the entry points do, without touching the GPU.  Returns
 * NCN_OK or the error the corresponding call would return before launching.  It takes no scalars: an entry point
 * additionally returns NCN_ERR_UNSUPPORTED when ncn_kernel_path_scalars(shape, alpha, m) is 0 (alpha or m outside the
 * range of the register kernels at a head width the generic kernels do not take).  No reference counterpart (the
 * reference validates nothing). */
int ncn_check_shape(const ncn_shape* shape, int first_stage, int n_stages, int activation);

/* Human-readable text for a code returned by the functions above. */
const char* ncn_error_string(int code);

/* Library version, "major.minor". */
const char* ncn_version(void);

/* Build id: 16 hex digits, a hash of every source file, header and compiler flag the library was made from.  The
 * Python loader compares it with the hash of the sources it finds beside the library and rebuilds when they differ
 * (file times play no part).  No reference counterpart. */
const char* ncn_build_id(void);

/* Measurement aid, no part of the layer and no reference counterpart: kernels that only issue one kind of vector
 * instruction, or a mix shaped like the step code of the NCN kernels, built like the rest of the library (no packed
 * FP32).  bench.py quotes the rate of a stream of v_fma_f32 on vector registers beside the published 157.3 TFLOP/s,
 * and `python -m ncn_cuda_amd.probe` prints the whole table.
 * ncn_probe_issue launches `waves_per_simd` (1, 2, 4, 8) workgroups of 256 threads per CU, one wave per SIMD each (the
 * dynamic LDS they ask for keeps a CU from taking more); every lane runs `chains` (1, 4, 8) independent dependency
 * chains of iters * G groups of instructions, G = the return value of ncn_probe_issue_info, which also gives the
 * vector instructions and the floating-point operations one group counts.  out: 8 * CUs * 256 floats.  The caller
 * times the launch with events on `stream`. */
#define NCN_PROBE_FMA 0           /* v_fma_f32, every source a vector register */
#define NCN_PROBE_ADD 1           /* v_add_f32, likewise */
#define NCN_PROBE_MUL 2           /* v_mul_f32, likewise */
#define NCN_PROBE_EXP2 3          /* v_exp_f32 */
#define NCN_PROBE_RCP 4           /* v_rcp_f32 */
#define NCN_PROBE_EXP2_ADD_RCP 5  /* 1 / (1 + 2^x): the activation of a step */
#define NCN_PROBE_DPP_ADD 6       /* v_add_f32 with a DPP quad_perm operand */
#define NCN_PROBE_SWIZZLE_ADD 7   /* ds_swizzle_b32 + v_add_f32 */
#define NCN_PROBE_BACKWARD_MIX 8  /* 13 fma, 4 add (2 across lanes), 1 mul, exp2, rcp: one element-step of the backward */
#define NCN_PROBE_FORWARD_MIX 9   /* 5 fma, 2 add (1 across lanes), exp2, rcp: one element-step of the forward */
#define NCN_PROBE_MFMA 10         /* v_mfma_f32_16x16x4_f32 */
#define NCN_PROBE_FMA_AND_MFMA 11 /* 4 v_fma_f32 and one independent v_mfma_f32_16x16x4_f32: do they overlap? */
#define NCN_PROBE_FMA_SGPR 12     /* v_fmac_f32 with a scalar-register source, every instruction */
#define NCN_PROBE_FMA_SGPR_1_IN_4 13 /* the same, three v_fma_f32 on vector registers between two of them */
#define NCN_PROBE_EXP2_1_IN_8 14  /* one v_exp_f32 and seven v_fma_f32: what a transcendental costs inside other work */
#define NCN_PROBE_DPP_1_IN_2 15   /* v_add_f32 with a DPP operand and v_fma_f32 in turns */
#define NCN_PROBE_MODES 16
int ncn_probe_issue(int mode, int chains, int waves_per_simd, int iters, float* out, void* stream);
int ncn_probe_issue_info(int mode, int* valu_per_group, int* flops_per_group);

#ifdef __cplusplus
}
#endif
#endif /* NCN_HIP_H */
