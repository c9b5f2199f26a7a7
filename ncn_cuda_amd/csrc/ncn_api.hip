// C ABI of libncn_hip.so: argument validation, stage sequencing and launches.  See include/ncn_hip.h.
#include <hip/hip_runtime.h>

#include <cmath>
#include <mutex>

#include "../../include/ncn_hip.h"
#include "ncn_fused_kernels.h"
#include "ncn_launch.h"

namespace {

using namespace ncn;

bool known_activation(int a) {
    return a == NCN_ACT_TANH || a == NCN_ACT_RELU || a == NCN_ACT_SIGMOID || a == NCN_ACT_LEAKY_RELU || a == NCN_ACT_LINEAR;
}
bool known_dtype(int d) { return d == NCN_F32 || d == NCN_BF16; }
// the arguments that also take a value kept as two bfloat16 planes (one stage per call, register kernels)
bool known_dtype_or_x2(int d, int n_stages, int path) { return known_dtype(d) || (d == NCN_BF16X2 && n_stages == 1 && path == 2); }
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Heads of one feature (E == n_head) run on the register kernels of ncn_headwise_kernels.h, four adjacent heads to a lane.
bool headwise_shape(const ncn_shape* sh) {
    const int w = headwise_width(sh->E);
    return sh->E == sh->n_head && w != 0 && sh->n_cache <= 64 && fast_tile(sh->n_cache, w).r != 0;
}

// 2 = register kernels, 1 = generic LDS kernels, 0 = unsupported
int kernel_path(const ncn_shape* sh, int /*activation*/) {
    if (sh->n_cache < 1 || sh->n_cache > 64) return 0;
    const int64_t ec = sh->E / sh->n_head;
    if (headwise_shape(sh)) return 2;
    if (ec <= 128 && fast_tile(sh->n_cache, (int)ec).r != 0) return 2;
    if (ec <= kGenericMaxHeadDim) return 1;
    return 0;
}

// The register kernels carry x times 2 log2(e) alpha and xa times that and (1-m) (StepTable): alpha, m and 1-m must
// stay away from zero.  Other values go to the generic kernels, which use the plain formulas.
bool scalars_fit_scaled_state(float alpha, float m) {
    return alpha >= 1e-3f && alpha <= 1e3f && m >= 1e-3f && m <= 1.0f - 1e-3f;
}

// kernel_path() for a call with these scalars: 2, 1, or 0 when nothing can run it
int kernel_path_for(const ncn_shape* sh, int activation, float alpha, float m) {
    const int path = kernel_path(sh, activation);
    if (path != 2 || scalars_fit_scaled_state(alpha, m)) return path;
    return (sh->E / sh->n_head <= kGenericMaxHeadDim) ? 1 : 0;
}

int check_shape(const ncn_shape* sh, int first_stage, int n_stages, int activation) {
    if (!sh) return NCN_ERR_NULL;
    if (sh->batch <= 0 || sh->N <= 0 || sh->E <= 0 || sh->n_head <= 0 || sh->n_cache <= 0) return NCN_ERR_SHAPE;
    if (sh->N % sh->n_cache != 0 || sh->E % sh->n_head != 0) return NCN_ERR_SHAPE;
    if (first_stage < 0 || n_stages < 1) return NCN_ERR_SHAPE;
    if (!known_activation(activation)) return NCN_ERR_ACTIVATION;
    if (kernel_path(sh, activation) == 0) return NCN_ERR_UNSUPPORTED;
    // 32-bit tile and block arithmetic inside the kernels
    const int64_t groups = sh->N / sh->n_cache;
    if (groups > (int64_t)1 << 24) return NCN_ERR_UNSUPPORTED;
    if (sh->batch * groups > (int64_t)1 << 30) return NCN_ERR_UNSUPPORTED;
    return NCN_OK;
}

// 2^(stage-1) mod groups without overflow (torch_ref/ncn_pytorch.py:38 uses Python big integers)
uint32_t stage_stride(int stage, uint32_t groups) {
    if (stage == 0) return 0;
    uint64_t r = 1 % groups, b = 2 % groups;
    for (uint32_t e = (uint32_t)stage - 1; e; e >>= 1) {   // square and multiply: any stage number costs 31 rounds
        if (e & 1) r = r * b % groups;
        b = b * b % groups;
    }
    return (uint32_t)r;
}

struct Plan {
    int path;
    int groups_per_tile;
    uint32_t groups, tiles_per_inst, total_tiles;
    int grid_x;        // backward launch
    int grid_fwd;      // forward / inverse launch
    int partial_rows;  // rows of the dW partial buffer the backward launch writes
};

// reserve_rows: rows of the dW partial buffer kept free for another launch of the same stage
// row_cap: rows of the dW partial buffer the caller has (kMaxGridX in a workspace of ncn_workspace_bytes)
Plan make_plan(const ncn_shape* sh, int path, int reserve_rows = 0, int row_cap = kMaxGridX) {
    Plan p;
    const int max_rows = row_cap - reserve_rows;
    p.path = path;
    const int ec = (int)(sh->E / sh->n_head);
    p.groups_per_tile = (p.path == 2) ? fast_groups_per_tile(sh->n_cache, ec) : generic_groups_per_tile(sh->n_cache);
    p.groups = (uint32_t)(sh->N / sh->n_cache);
    p.tiles_per_inst = (p.groups + p.groups_per_tile - 1) / p.groups_per_tile;
    p.total_tiles = (uint32_t)(sh->batch * p.tiles_per_inst);
    if (p.path == 2) {
        // 4 waves per block, wave w works on head w % n_head: the grid holds a multiple of n_head waves and at
        // most kMaxGridX partial rows (one per n_head consecutive waves)
        const int C = sh->n_head;
        const int g4 = (C % 4 == 0) ? 4 : (C % 2 == 0 ? 2 : 1);
        const int64_t quantum = C / g4;                                   // blocks per multiple of n_head waves
        const int64_t cap = (int64_t)max_rows * C / 4 / quantum * quantum;  // rows = blocks * 4 / C <= max_rows
        int64_t blocks = ((int64_t)p.total_tiles * C + 3) / 4;
        blocks = (blocks + quantum - 1) / quantum * quantum;
        // forward / inverse write no partials: one wave tile per wave where possible (measured 8 % faster than a
        // persistent loop over 4096 blocks: retiring blocks balance the load)
        int64_t fblocks = blocks;
        const int64_t fcap = (int64_t)kMaxForwardGridX / quantum * quantum;
        if (fblocks > fcap) fblocks = fcap;
        if (fblocks < quantum) fblocks = quantum;
        p.grid_fwd = (int)fblocks;
        if (blocks > cap) blocks = cap;
        if (blocks < quantum) blocks = quantum;
        p.grid_x = (int)blocks;
        p.partial_rows = (int)(blocks * 4 / C);
    } else {
        p.grid_x = (int)(p.total_tiles < (uint32_t)max_rows ? p.total_tiles : (uint32_t)max_rows);
        p.grid_fwd = p.grid_x;
        p.partial_rows = p.grid_x;
    }
    return p;
}

void fill_step_table(StepTable& t, int n_cache, float alpha, float m, int activation = NCN_ACT_TANH) {
    // a call fills the same table for every stage it launches, and callers repeat (alpha, m) step after step:
    // keep the last one per thread (some 70 pow() otherwise)
    thread_local StepTable cached;
    thread_local int cached_n = -1;
    if (cached_n == n_cache && cached.alpha == alpha && cached.m == m) {
        t = cached;
        t.activation = activation;
        return;
    }
    const double md = m, al = alpha, k2l = 2.8853900817779268, om = 1.0 - md, im = 1.0 / md;
    // the generic kernels read alpha and m only; for scalars that do not fit the scaled state the rest stays finite
    const bool fit = scalars_fit_scaled_state(alpha, m);
    const double kappa = fit ? k2l * al : 1.0, ks = fit ? kappa * om : 1.0;
    t.alpha = alpha;
    t.m = m;
    t.activation = activation;
    t.reserved = 0;
    t.kappa = (float)kappa;
    t.inv_kappa = (float)(1.0 / kappa);
    t.a_scale = (float)ks;
    t.inv_a_scale = (float)(1.0 / ks);
    t.b_scale = (float)(ks * im);
    t.inv_b_scale = (float)(md / ks);
    t.gamma = (float)(fit ? (1.0 - al) / (k2l * al * al) : 0.0);
    t.om = (float)om;
    t.im = (float)im;
    const double k2 = kappa * om * om;
    t.k2 = (float)k2;
    t.m2k2 = (float)(-2.0 * k2);
    t.bk0 = (float)(-k2 * im * im);
    t.bk1 = (float)(2.0 * k2 * im * im);
    t.ku = (float)(4.0 * om * al * im);
    t.m_pow_n = (float)std::pow(md, (double)n_cache);
    t.inv_m_pow_n = (float)std::pow(md, -(double)n_cache);
    t.reserved2 = 0.f;
    for (int k = 0; k < 64; ++k) t.krho[k] = (float)((1.0 - al) * 4.0 * om * std::pow(md, (double)k) / (kappa * kappa));
    cached = t;
    cached_n = n_cache;
}

// How the rows are grouped and which of them are live: caller's tables of the *_indexed entry points, or nothing.
struct Grouping {
    const int32_t* table;    // [n_stages, N] or null
    const int32_t* ctx_len;  // [batch] or null
    int radix_first = -1;    // >= 0: stage k is radix level radix_first + k (no table then)
    bool plain() const { return !table && !ctx_len && radix_first < 0; }
    bool permutation() const { return !table && radix_first < 0; }   // the stride permutation, with or without lengths
};

uint32_t upow(uint32_t b, int e) {
    uint64_t r = 1;
    for (int k = 0; k < e; ++k) r *= b;
    return (uint32_t)r;
}

// levels first .. first+count-1 exist when n^(first+count) divides N
int check_radix(const ncn_shape* sh, int first, int count) {
    if (first < 0 || count < 1) return NCN_ERR_SHAPE;
    int64_t p = 1;
    for (int k = 0; k < first + count; ++k) {
        p *= sh->n_cache;
        if (p > sh->N) return NCN_ERR_SHAPE;
    }
    return (sh->N % p == 0) ? NCN_OK : NCN_ERR_SHAPE;
}

int check_grouping(const Grouping& g, const ncn_shape* sh) {
    if ((reinterpret_cast<uintptr_t>(g.table) & 3u) || (reinterpret_cast<uintptr_t>(g.ctx_len) & 3u)) return NCN_ERR_ALIGN;
    (void)sh;
    return NCN_OK;
}

void fill_common(StageArgs& a, const ncn_shape* sh, const Plan& p, int stage, float alpha, float m, int activation,
                 const Grouping& g = Grouping{nullptr, nullptr}, int rel_stage = 0) {
    a.table = g.table ? g.table + (int64_t)rel_stage * sh->N : nullptr;
    a.ctx_len = g.ctx_len;
    a.edge = 0;
    a.radix_stride = g.radix_first >= 0 ? upow((uint32_t)sh->n_cache, g.radix_first + rel_stage) : 0u;
    a.N = sh->N;
    a.E = sh->E;
    a.plane = sh->batch * sh->N * sh->E;
    a.total_tiles = p.total_tiles;
    a.tiles_per_inst = p.tiles_per_inst;
    a.groups = p.groups;
    a.stride = stage_stride(stage, p.groups);
    a.groups_pow2 = (p.groups & (p.groups - 1)) == 0 ? 1u : 0u;
    a.n_cache = sh->n_cache;
    a.head_dim = (int)(sh->E / sh->n_head);
    a.n_head = sh->n_head;
    a.activation = activation;
    fill_step_table(a.tab, sh->n_cache, alpha, m, activation);
}

// With context lengths, after the main launch: the rows past the lengths pass through.  The register kernels run
// the group a length cuts themselves (masked steps); the generic kernel leaves it to a second launch of its own,
// one tile per batch entry.  `a` is the stage's argument block as the main launch used it.
hipError_t launch_ragged_rest(Pass pass, StageArgs a, const ncn_shape* sh, int path, int partial_rows_used,
                              hipStream_t s) {
    if (path != 2) {
        StageArgs e = a;
        e.edge = 1;
        e.total_tiles = (uint32_t)sh->batch;
        e.tiles_per_inst = 1;
        if (pass == kBackward) e.dw_partials = a.dw_partials + (int64_t)partial_rows_used * 2 * sh->E;
        const int grid = (int)(sh->batch < kEdgeGridX ? sh->batch : kEdgeGridX);
        hipError_t err = launch_generic(pass, e, sh->n_head, grid, s);
        if (err != hipSuccess) return err;
    }
    return launch_pass_through(pass, a, sh->batch, s);
}
int edge_rows(const ncn_shape* sh) { return (int)(sh->batch < kEdgeGridX ? sh->batch : kEdgeGridX); }

// A call on heads of one feature that the register kernels take (path 2) is planned and launched with the geometry
// of E / w heads of w = headwise_width(E) features, which `as_wide` receives: same tiles, grids and partial rows as
// for such heads, other kernels.
bool headwise_call(const ncn_shape* sh, int path, ncn_shape* as_wide) {
    if (path != 2 || !headwise_shape(sh)) return false;
    *as_wide = *sh;
    as_wide->n_head = (int)(sh->E / headwise_width(sh->E));
    return true;
}

// the shape that the passes of a call on `sh` are planned for (the queries take no scalars: register kernels assumed)
const ncn_shape* planning_shape(const ncn_shape* sh, ncn_shape* as_wide) {
    return headwise_call(sh, 2, as_wide) ? as_wide : sh;
}

// one stage on the register kernels: the plain builds know the stride permutation only, the others read the
// launch's table, radix level and context lengths
hipError_t run_forward_kernel(Pass pass, const StageArgs& a, bool plain, bool headwise, int n_head, int grid,
                              hipStream_t s) {
    if (headwise) return plain ? launch_headwise_forward(pass, a, grid, s) : launch_headwise_forward_indexed(pass, a, grid, s);
    return plain ? launch_fast_forward(pass, a, n_head, grid, s) : launch_fast_forward_indexed(pass, a, n_head, grid, s);
}
hipError_t run_backward_kernel(const StageArgs& a, bool plain, bool headwise, int n_head, int grid, hipStream_t s) {
    if (headwise) return plain ? launch_headwise_backward(a, grid, s) : launch_headwise_backward_indexed(a, grid, s);
    return plain ? launch_fast_backward(a, n_head, grid, s) : launch_fast_backward_indexed(a, n_head, grid, s);
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// rows of chunk sums that the launches of one reduction job can need when they fill row_cap partial rows
int level1_rows(int row_cap) {
    const int r = row_cap / kReduceRowsPerBlock + kReduceMaxStages;
    return r > kReduceLevel1Rows ? r : kReduceLevel1Rows;
}
// dW partial rows of the backward launches of a call, then the chunk sums of the first reduction level
size_t partial_buffer_bytes(const ncn_shape* sh, int row_cap) {
    return align256((size_t)(row_cap + level1_rows(row_cap)) * 2 * (size_t)sh->E * sizeof(float));
}
size_t base_workspace_bytes(const ncn_shape* sh) { return partial_buffer_bytes(sh, kMaxGridX); }

// the multi-stage plan of a stage range, or an empty vector when the one-stage loop should be used
std::vector<FusedPass> multi_stage_plan(const ncn_shape* sh, int first_stage, int n_stages, int activation, bool backward,
                                        int path = 2) {
    std::vector<FusedPass> none;
    if (n_stages < 2 || path != 2 || kernel_path(sh, activation) != 2 || !fused_supported(sh, activation)) return none;
    std::vector<FusedPass> passes = plan_fused(sh, first_stage, n_stages, backward);
    bool any = false;
    for (const FusedPass& p : passes) any = any || !p.single;
    return any ? passes : none;
}

// Partial rows that the backward passes of a plan fill when every window has a workgroup of its own (rows * stages,
// summed over the passes, which lie side by side in the buffer), between what every workspace holds and
// kFusedRowCapMax (64 MB at E = 128).
constexpr int kFusedRowCapMax = 65536;
int fused_rows_wanted(const ncn_shape* sh, const std::vector<FusedPass>& passes) {
    int64_t rows = 0;
    for (const FusedPass& p : passes)
        rows += p.single ? (int64_t)kMaxGridX : fused_items(sh, p) / sh->n_head * p.count;
    if (rows > kFusedRowCapMax) rows = kFusedRowCapMax;
    return rows < kMaxGridX ? kMaxGridX : (int)rows;
}

size_t temp_bytes(const ncn_shape* sh, bool backward) {
    return align256((size_t)sh->batch * sh->N * sh->E * sizeof(float)) * (backward ? 4 : 2);
}

// The backward launches of one call write their dW partial rows side by side into the partial buffer and are summed
// together: two reduction launches per call instead of two per launch, as long as the buffer (kMaxGridX rows of 2E)
// and the job (kReduceMaxSegments launches, kReduceMaxStages stages) hold them.
class DwReducer {
  public:
    DwReducer(float* partials, float* level1, int64_t two_e, hipStream_t s, int row_cap = kMaxGridX)
        : partials_(partials), level1_(level1), two_e_(two_e), stream_(s), row_cap_(row_cap) { job_.n = 0; }
    // Where a launch of `rows` partial rows of `stages` stages each may write; earlier launches are summed first
    // if it would not fit behind them.
    hipError_t reserve(int rows, int stages, float** region) {
        hipError_t err = hipSuccess;
        if (job_.n == kReduceMaxSegments || stages_ + stages > kReduceMaxStages ||
            used_rows_ + (int64_t)rows * stages > row_cap_)
            err = flush();
        *region = partials_ + used_rows_ * two_e_;
        return err;
    }
    // The launch that got `region` from reserve() has been enqueued: its column sums go to dW_out[stages * 2E].
    void add(const float* region, int rows, int stages, float* dW_out) {
        ReduceSegment& g = job_.seg[job_.n];
        g.in = region;
        g.out = dW_out;
        g.cols = stages * two_e_;
        g.rows = rows;
        g.chunk0 = chunks_;
        g.level1_offset = level1_floats_;
        const int chunks = (rows + kReduceRowsPerBlock - 1) / kReduceRowsPerBlock;
        chunks_ += chunks;
        level1_floats_ += (int64_t)chunks * g.cols;
        used_rows_ += (int64_t)rows * stages;
        stages_ += stages;
        ++job_.n;
    }
    hipError_t flush() {
        const hipError_t err = launch_reduce_job(job_, level1_, stream_);
        job_.n = 0;
        used_rows_ = level1_floats_ = 0;
        stages_ = chunks_ = 0;
        return err;
    }

  private:
    float* partials_;
    float* level1_;
    int64_t two_e_;
    hipStream_t stream_;
    ReduceJob job_;
    int row_cap_;
    int64_t used_rows_ = 0, level1_floats_ = 0;
    int stages_ = 0, chunks_ = 0;
};

// ---- scratch of ncn_backward_static: device memory that belongs to the library, one copy per GPU -----------------
// Holds the dW partial rows and chunk sums that ncn_backward takes from its workspace argument.  kStaticRowCap partial
// rows (a quarter of what a workspace gives: large problems loop over them) of up to kStaticMaxTwoE floats.
constexpr int kStaticRowCap = 4096;
constexpr int kStaticMaxTwoE = 512;
constexpr size_t kStaticScratchFloats = (size_t)(kStaticRowCap + kReduceLevel1Rows) * kStaticMaxTwoE;   // 9.0 MiB
constexpr int kStaticMaxDevices = 64;

}  // namespace

static __device__ __align__(256) float ncn_static_scratch[kStaticScratchFloats];

namespace {

// Address of the array on the current device.  The array's name is only a host-side handle: the address a kernel
// can use comes from hipGetSymbolAddress, once per device (every GPU holds its own copy at its own address).
hipError_t static_scratch(float** out) {
    static float* ptrs[kStaticMaxDevices] = {};
    static std::mutex lock;
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    if (dev < 0 || dev >= kStaticMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (!ptrs[dev]) {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(ncn_static_scratch));
        if (err != hipSuccess) return err;
        ptrs[dev] = static_cast<float*>(p);
    }
    *out = ptrs[dev];
    return hipSuccess;
}

}  // namespace

extern "C" {

const char* ncn_version(void) { return "0.15"; }

int ncn_plan_passes(const ncn_shape* shape, int first_stage, int n_stages, int activation, int backward, int32_t* out,
                    int max_passes) {
    int rc = check_shape(shape, first_stage, n_stages, activation);
    if (rc != NCN_OK) return rc;
    ncn_shape as_wide;
    shape = planning_shape(shape, &as_wide);
    const std::vector<FusedPass> passes = multi_stage_plan(shape, first_stage, n_stages, activation, backward != 0);
    int k = 0;
    for (const FusedPass& p : passes) {
        if (out && k < max_passes) {
            int32_t* o = out + 8 * k;
            o[0] = p.first; o[1] = p.count; o[2] = p.single ? 0 : (p.closed ? 2 : 1);
            o[3] = (int32_t)p.class_stride; o[4] = (int32_t)p.window; o[5] = (int32_t)p.halo; o[6] = (int32_t)p.own;
            o[7] = (int32_t)p.class_groups;
        }
        ++k;
    }
    return k;
}

const char* ncn_error_string(int code) {
    switch (code) {
        case NCN_OK: return "ok";
        case NCN_ERR_NULL: return "a required pointer is NULL";
        case NCN_ERR_SHAPE: return "bad shape: sizes must be positive, N % n_cache == 0, E % n_head == 0, n_stages >= 1";
        case NCN_ERR_DTYPE: return "unknown element type (0 = float32, 1 = bfloat16; 2 = two bfloat16 planes, only for the saved outputs of one stage on the register kernels)";
        case NCN_ERR_ACTIVATION: return "unknown activation code (0 tanh, 1 relu, 2 sigmoid, 3 leaky relu, -1 linear)";
        case NCN_ERR_WORKSPACE: return "workspace is NULL or smaller than ncn_workspace_bytes()";
        case NCN_ERR_UNSUPPORTED: return "unsupported shape: n_cache must be <= 64 and the head width <= 64 (128 for power-of-two n_cache <= 16)";
        case NCN_ERR_ALIGN: return "a pointer is not 16-byte aligned (4-byte for group_index and ctx_len)";
        case NCN_ERR_ALIAS: return "n_stages > 1 needs float32 dx, dxa and either x_rec, xa_rec or the workspace of ncn_workspace_bytes_stages(.., 2) to carry the state";
        case NCN_ERR_STATIC_LIMIT: return "ncn_backward_static: E is above 256, the limit of the library's own scratch";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

int ncn_check_shape(const ncn_shape* shape, int first_stage, int n_stages, int activation) {
    return check_shape(shape, first_stage, n_stages, activation);
}

int ncn_kernel_path(const ncn_shape* shape) {
    if (!shape || shape->batch <= 0 || shape->N <= 0 || shape->E <= 0 || shape->n_head <= 0 || shape->n_cache <= 0)
        return 0;
    if (shape->E % shape->n_head != 0) return 0;
    return kernel_path(shape, NCN_ACT_TANH);
}

int ncn_kernel_path_scalars(const ncn_shape* shape, float alpha, float m) {
    return ncn_kernel_path(shape) ? kernel_path_for(shape, NCN_ACT_TANH, alpha, m) : 0;
}

size_t ncn_workspace_bytes(const ncn_shape* shape) {
    if (check_shape(shape, 0, 1, NCN_ACT_TANH) != NCN_OK) return 0;
    return base_workspace_bytes(shape);
}

size_t ncn_workspace_bytes_stages(const ncn_shape* shape, int first_stage, int n_stages, int activation, int backward) {
    if (check_shape(shape, first_stage, n_stages, activation) != NCN_OK) return 0;
    ncn_shape as_wide;
    shape = planning_shape(shape, &as_wide);
    const std::vector<FusedPass> passes = multi_stage_plan(shape, first_stage, n_stages, activation, backward != 0);
    const size_t base = !backward ? 0 : passes.empty() ? base_workspace_bytes(shape)
                                                        : partial_buffer_bytes(shape, fused_rows_wanted(shape, passes));
    // backward == 2: the call will pass no x_rec, xa_rec, so the two arrays that carry the reconstructed state from
    // stage to stage come out of the workspace (a single pass over closed rings carries nothing; a single halo pass
    // may have to give way to one launch per stage when the caller's buffers alias, and those carry)
    const bool one_closed_pass = passes.size() == 1 && passes[0].closed && !passes[0].single;
    const size_t carriers = (backward == 2 && n_stages > 1 && !one_closed_pass) ? temp_bytes(shape, true) / 2 : 0;
    return (passes.size() >= 2 ? base + temp_bytes(shape, backward != 0) : base) + carriers;
}

static int forward_impl(const void* x, const void* xa, int in_dtype, void* y, void* ya, int out_dtype, float* y32,
                        float* ya32, const float* W, void* workspace, size_t workspace_bytes, const Grouping& grouping,
                        const ncn_shape* shape, int first_stage, int n_stages, float alpha, float m, int activation,
                        void* stream) {
    int rc = check_shape(shape, first_stage, n_stages, activation);
    if (rc != NCN_OK) return rc;
    rc = check_grouping(grouping, shape);
    if (rc != NCN_OK) return rc;
    if (!x || !xa || !y || !ya || !W) return NCN_ERR_NULL;
    if ((y32 == nullptr) != (ya32 == nullptr)) return NCN_ERR_NULL;
    const int path = kernel_path_for(shape, activation, alpha, m);
    if (path == 0) return NCN_ERR_UNSUPPORTED;
    ncn_shape as_wide;
    const bool headwise = headwise_call(shape, path, &as_wide);
    if (headwise) shape = &as_wide;
    if (!known_dtype(in_dtype) || !known_dtype_or_x2(out_dtype, n_stages, path)) return NCN_ERR_DTYPE;
    if (!aligned16(x) || !aligned16(xa) || !aligned16(y) || !aligned16(ya) || !aligned16(W) || !aligned16(y32) ||
        !aligned16(ya32) || !aligned16(workspace))
        return NCN_ERR_ALIGN;
    const Plan p = make_plan(shape, path);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t wstride = 2 * shape->E;

    // several stages: LDS-resident passes when the shape allows and the buffers permit the ping-pong
    std::vector<FusedPass> passes;
    if (grouping.permutation()) passes = multi_stage_plan(shape, first_stage, n_stages, activation, false, path);
    const size_t np = passes.size();
    // one stage of the range with the one-stage kernel (and, with lengths, the launch for the rows past them)
    auto run_stage = [&](int k, const void* i0, const void* i1, int i_dtype, void* o0, void* o1, int o_dtype,
                         bool with_copies) -> hipError_t {
        StageArgs a{};
        fill_common(a, shape, p, first_stage + k, alpha, m, activation, grouping, k);
        a.in0 = i0; a.in1 = i1; a.in_dtype = i_dtype;
        a.out0 = o0; a.out1 = o1; a.out_dtype = o_dtype;
        a.aux0 = with_copies ? y32 : nullptr; a.aux1 = with_copies ? ya32 : nullptr;
        a.W = W + k * wstride;
        hipError_t err = run_forward_kernel(kForward, a, grouping.plain(), headwise, shape->n_head, p.grid_fwd, s);
        if (err == hipSuccess && grouping.ctx_len) err = launch_ragged_rest(kForward, a, shape, p.path, 0, s);
        return err;
    };
    bool fused_ok = np > 0 && (np < 2 || out_dtype == NCN_F32);
    // Buffers in turns (scratch and y, ya) when the scratch is there; a halo pass (or a one-stage launch feeding one)
    // must not write where another workgroup still reads its halo, so not when the first pass would write straight
    // into x, xa.  Otherwise the first pass goes from x, xa to y, ya and the others work in place on y, ya, where the
    // stages of a halo pass run one launch each (closed passes and one-stage launches may work in place).
    const bool turns = fused_ok && (np < 2 || (workspace && workspace_bytes >= temp_bytes(shape, false))) &&
                       !((x == y || xa == ya) && ((np - 1) % 2) == 0 && !passes[0].closed && !passes[0].single);
    if (fused_ok && !turns) {
        for (size_t k = 0; k < np; ++k) {
            const FusedPass& ps = passes[k];
            const bool last = (k + 1 == np);
            const bool in_place = k > 0 || x == y || xa == ya;
            hipError_t err = hipSuccess;
            if (ps.single || (!ps.closed && in_place)) {
                for (int j = ps.first; j < ps.first + ps.count && err == hipSuccess; ++j) {
                    const bool from_x = (k == 0 && j == ps.first);
                    err = run_stage(j, from_x ? x : y, from_x ? xa : ya, from_x ? in_dtype : out_dtype, y, ya, out_dtype,
                                    last && j == ps.first + ps.count - 1);
                }
            } else {
                FusedArgs a{};
                a.in0 = k == 0 ? x : y; a.in1 = k == 0 ? xa : ya; a.in_dtype = k == 0 ? in_dtype : out_dtype;
                a.out0 = y; a.out1 = ya; a.out_dtype = out_dtype;
                a.aux0 = last ? y32 : nullptr; a.aux1 = last ? ya32 : nullptr;
                a.W = W + ps.first * wstride;
                a.ctx_len = grouping.ctx_len;
                fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
                err = launch_fused(kForward, a, shape, ps, s, kMaxGridX, headwise);
            }
            if (err != hipSuccess) return (int)err;
        }
        return NCN_OK;
    }
    if (turns) {
        const size_t one = temp_bytes(shape, false) / 2;
        void* t0 = workspace;
        void* t1 = workspace ? static_cast<char*>(workspace) + one : nullptr;
        const void* cur0 = x;
        const void* cur1 = xa;
        int cur_dtype = in_dtype;
        for (size_t k = 0; k < np; ++k) {
            const FusedPass& ps = passes[k];
            const bool to_out = ((np - 1 - k) % 2) == 0;
            const bool last = (k + 1 == np);
            void* d0 = to_out ? y : t0;
            void* d1 = to_out ? ya : t1;
            const int d_dtype = to_out ? out_dtype : NCN_F32;
            hipError_t err;
            if (ps.single) {
                err = run_stage(ps.first, cur0, cur1, cur_dtype, d0, d1, d_dtype, last);
            } else {
                FusedArgs a{};
                a.in0 = cur0; a.in1 = cur1; a.in_dtype = cur_dtype;
                a.out0 = d0; a.out1 = d1; a.out_dtype = d_dtype;
                a.aux0 = last ? y32 : nullptr; a.aux1 = last ? ya32 : nullptr;
                a.W = W + ps.first * wstride;
                a.ctx_len = grouping.ctx_len;
                fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
                err = launch_fused(kForward, a, shape, ps, s, kMaxGridX, headwise);
            }
            if (err != hipSuccess) return (int)err;
            cur0 = d0; cur1 = d1; cur_dtype = d_dtype;
        }
        return NCN_OK;
    }

    for (int k = 0; k < n_stages; ++k) {
        StageArgs a{};
        fill_common(a, shape, p, first_stage + k, alpha, m, activation, grouping, k);
        a.in0 = k == 0 ? x : y;
        a.in1 = k == 0 ? xa : ya;
        a.in_dtype = k == 0 ? in_dtype : out_dtype;
        a.out0 = y;
        a.out1 = ya;
        a.out_dtype = out_dtype;
        const bool last = (k == n_stages - 1);
        a.aux0 = last ? y32 : nullptr;
        a.aux1 = last ? ya32 : nullptr;
        a.W = W + k * wstride;
        hipError_t err = (p.path != 2) ? launch_generic(kForward, a, shape->n_head, p.grid_fwd, s)
                                       : run_forward_kernel(kForward, a, grouping.plain(), headwise, shape->n_head, p.grid_fwd, s);
        if (err == hipSuccess && grouping.ctx_len) err = launch_ragged_rest(kForward, a, shape, p.path, 0, s);
        if (err != hipSuccess) return (int)err;
    }
    return NCN_OK;
}

static int inverse_impl(const void* y, const void* ya, int in_dtype, void* x, void* xa, int out_dtype, const float* W,
                        void* workspace, size_t workspace_bytes, const Grouping& grouping, const ncn_shape* shape, int first_stage, int n_stages, float alpha,
                        float m, int activation, void* stream) {
    int rc = check_shape(shape, first_stage, n_stages, activation);
    if (rc != NCN_OK) return rc;
    rc = check_grouping(grouping, shape);
    if (rc != NCN_OK) return rc;
    if (!x || !xa || !y || !ya || !W) return NCN_ERR_NULL;
    const int path = kernel_path_for(shape, activation, alpha, m);
    if (path == 0) return NCN_ERR_UNSUPPORTED;
    ncn_shape as_wide;
    const bool headwise = headwise_call(shape, path, &as_wide);
    if (headwise) shape = &as_wide;
    if (!known_dtype_or_x2(in_dtype, n_stages, path) || !known_dtype(out_dtype)) return NCN_ERR_DTYPE;
    if (!aligned16(x) || !aligned16(xa) || !aligned16(y) || !aligned16(ya) || !aligned16(W) || !aligned16(workspace))
        return NCN_ERR_ALIGN;
    const Plan p = make_plan(shape, path);
    hipStream_t s = static_cast<hipStream_t>(stream);

    // several stages: LDS-resident passes, last pass of the range first.  Without scratch to ping-pong with, the
    // first pass to run goes from y, ya to x, xa and the others work in place on x, xa, which a halo pass must not,
    // so the stages of such a pass are undone by one-stage launches (closed passes and one-stage launches may).
    std::vector<FusedPass> passes;
    if (grouping.permutation() && (out_dtype == NCN_F32 || n_stages == 1))
        passes = multi_stage_plan(shape, first_stage, n_stages, activation, false, path);
    auto run_stage = [&](int k, const void* i0, const void* i1, int i_dtype, void* o0, void* o1, int o_dtype) -> hipError_t {
        StageArgs a{};
        fill_common(a, shape, p, first_stage + k, alpha, m, activation, grouping, k);
        a.in0 = i0; a.in1 = i1; a.in_dtype = i_dtype;
        a.out0 = o0; a.out1 = o1; a.out_dtype = o_dtype;
        a.W = W + (int64_t)k * 2 * shape->E;
        hipError_t err = run_forward_kernel(kInverse, a, grouping.plain(), headwise, shape->n_head, p.grid_fwd, s);
        if (err == hipSuccess && grouping.ctx_len) err = launch_ragged_rest(kInverse, a, shape, p.path, 0, s);
        return err;
    };
    // With scratch every pass reads one pair of buffers and writes another (scratch and x, xa in turns, so that the
    // last pass to run lands in x, xa), as the forward does, and every multi-stage pass runs as one.
    const bool ping_pong = passes.size() >= 2 && out_dtype == NCN_F32 && workspace &&
                           workspace_bytes >= temp_bytes(shape, false) &&
                           !((x == y || xa == ya) && ((passes.size() - 1) % 2) == 0);   // never straight from y into y
    if (ping_pong) {
        const int64_t wstride = 2 * shape->E;
        const size_t np = passes.size();
        const size_t one = temp_bytes(shape, false) / 2;
        void* t0 = workspace;
        void* t1 = static_cast<char*>(workspace) + one;
        const void* cur0 = y;
        const void* cur1 = ya;
        int cur_dtype = in_dtype;
        for (size_t e = 0; e < np; ++e) {
            const FusedPass& ps = passes[np - 1 - e];
            const bool to_out = ((np - 1 - e) % 2) == 0;
            void* d0 = to_out ? x : t0;
            void* d1 = to_out ? xa : t1;
            hipError_t err;
            if (ps.single) {
                err = run_stage(ps.first, cur0, cur1, cur_dtype, d0, d1, NCN_F32);
            } else {
                FusedArgs a{};
                a.in0 = cur0; a.in1 = cur1; a.in_dtype = cur_dtype;
                a.out0 = d0; a.out1 = d1; a.out_dtype = NCN_F32;
                a.W = W + ps.first * wstride;
                a.ctx_len = grouping.ctx_len;
                fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
                err = launch_fused(kInverse, a, shape, ps, s, kMaxGridX, headwise);
            }
            if (err != hipSuccess) return (int)err;
            cur0 = d0; cur1 = d1; cur_dtype = NCN_F32;
        }
        return NCN_OK;
    }
    if (!passes.empty()) {
        const int64_t wstride = 2 * shape->E;
        const size_t np = passes.size();
        for (size_t e = 0; e < np; ++e) {
            const FusedPass& ps = passes[np - 1 - e];
            const bool top = (e == 0);
            const bool in_place = !top || x == y || xa == ya;
            if (ps.single || (!ps.closed && in_place)) {
                for (int k = ps.first + ps.count - 1; k >= ps.first; --k) {
                    const bool from_y = top && k == ps.first + ps.count - 1;
                    hipError_t err = run_stage(k, from_y ? y : x, from_y ? ya : xa, from_y ? in_dtype : out_dtype, x, xa,
                                               out_dtype);
                    if (err != hipSuccess) return (int)err;
                }
            } else {
                FusedArgs a{};
                a.in0 = top ? y : x; a.in1 = top ? ya : xa; a.in_dtype = top ? in_dtype : out_dtype;
                a.out0 = x; a.out1 = xa; a.out_dtype = out_dtype;
                a.W = W + ps.first * wstride;
                a.ctx_len = grouping.ctx_len;
                fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
                hipError_t err = launch_fused(kInverse, a, shape, ps, s, kMaxGridX, headwise);
                if (err != hipSuccess) return (int)err;
            }
        }
        return NCN_OK;
    }

    for (int k = n_stages - 1; k >= 0; --k) {
        StageArgs a{};
        fill_common(a, shape, p, first_stage + k, alpha, m, activation, grouping, k);
        const bool first = (k == n_stages - 1);
        a.in0 = first ? y : x;
        a.in1 = first ? ya : xa;
        a.in_dtype = first ? in_dtype : out_dtype;
        a.out0 = x;
        a.out1 = xa;
        a.out_dtype = out_dtype;
        a.W = W + (int64_t)k * 2 * shape->E;
        hipError_t err = (p.path != 2) ? launch_generic(kInverse, a, shape->n_head, p.grid_fwd, s)
                                       : run_forward_kernel(kInverse, a, grouping.plain(), headwise, shape->n_head, p.grid_fwd, s);
        if (err == hipSuccess && grouping.ctx_len) err = launch_ragged_rest(kInverse, a, shape, p.path, 0, s);
        if (err != hipSuccess) return (int)err;
    }
    return NCN_OK;
}

static int backward_impl(const void* y, const void* ya, int y_dtype, const void* dy, const void* dya, int dy_dtype,
                         void* dx, void* dxa, int dx_dtype, float* x_rec, float* xa_rec, const float* W, float* dW,
                         void* workspace, size_t workspace_bytes, const Grouping& grouping, const ncn_shape* shape,
                         int first_stage, int n_stages, float alpha, float m, int activation, void* stream,
                         int row_cap = kMaxGridX) {
    int rc = check_shape(shape, first_stage, n_stages, activation);
    if (rc != NCN_OK) return rc;
    rc = check_grouping(grouping, shape);
    if (rc != NCN_OK) return rc;
    if (!y || !ya || !dy || !dx || !dxa || !W || !dW) return NCN_ERR_NULL;
    if ((x_rec == nullptr) != (xa_rec == nullptr)) return NCN_ERR_NULL;
    const int path = kernel_path_for(shape, activation, alpha, m);
    if (path == 0) return NCN_ERR_UNSUPPORTED;
    ncn_shape as_wide;
    const bool headwise = headwise_call(shape, path, &as_wide);
    if (headwise) shape = &as_wide;
    if (!known_dtype_or_x2(y_dtype, n_stages, path) || !known_dtype(dy_dtype) || !known_dtype(dx_dtype)) return NCN_ERR_DTYPE;
    if (n_stages > 1 && dx_dtype != NCN_F32) return NCN_ERR_ALIAS;
    if (!workspace || workspace_bytes < partial_buffer_bytes(shape, row_cap)) return NCN_ERR_WORKSPACE;
    // Several stages without x_rec, xa_rec: the caller does not want the reconstructed inputs.  The stages before the
    // last one to run still hand their reconstructed inputs on, through two arrays taken from the end of the
    // workspace (ncn_workspace_bytes_stages(.., backward = 2)); the last one does not write them at all.
    const bool no_rec = n_stages > 1 && !x_rec;
    const size_t plane_bytes = temp_bytes(shape, true) / 4;
    if (!aligned16(y) || !aligned16(ya) || !aligned16(dy) || !aligned16(dya) || !aligned16(dx) || !aligned16(dxa) ||
        !aligned16(x_rec) || !aligned16(xa_rec) || !aligned16(W) || !aligned16(dW) || !aligned16(workspace))
        return NCN_ERR_ALIGN;
    // partial rows of the generic kernel's second launch
    const int extra_rows = (grouping.ctx_len && path != 2) ? edge_rows(shape) : 0;
    const Plan p = make_plan(shape, path, extra_rows, row_cap);
    hipStream_t s = static_cast<hipStream_t>(stream);
    float* partials = static_cast<float*>(workspace);
    float* level1 = partials + (int64_t)row_cap * 2 * shape->E;
    const int64_t wstride = 2 * shape->E;

    // several stages: LDS-resident passes, last pass of the range first; the state ping-pongs between the
    // output arrays and four float32 arrays behind the dW scratch (their grids count on kMaxGridX partial rows)
    std::vector<FusedPass> passes;
    if (grouping.permutation() && row_cap == kMaxGridX)
        passes = multi_stage_plan(shape, first_stage, n_stages, activation, true, path);
    const size_t np = passes.size();
    bool fused_ok = np > 0;
    // a workspace of ncn_workspace_bytes_stages() holds a partial row for every window of every pass; a smaller one
    // (ncn_workspace_bytes() and the four arrays) makes the workgroups loop over windows
    int fused_cap = kMaxGridX;
    const size_t fused_extra = np >= 2 ? temp_bytes(shape, true) + (no_rec ? 2 * plane_bytes : 0) : 0;
    if (np > 0) {
        const int want = fused_rows_wanted(shape, passes);
        if (workspace_bytes >= partial_buffer_bytes(shape, want) + fused_extra) fused_cap = want;
    }
    const size_t fused_base = partial_buffer_bytes(shape, fused_cap);
    if (np >= 2 && workspace_bytes < fused_base + fused_extra) fused_ok = false;
    if (np >= 1 && ((np - 1) % 2) == 0 && !passes[np - 1].closed && !passes[np - 1].single &&
        (y == x_rec || ya == xa_rec || dy == dx || (dya && dya == dxa)))
        fused_ok = false;  // the first pass to run is a halo pass and would write into its own input
    if (fused_ok) {
        const size_t one = temp_bytes(shape, true) / 4;
        char* tb = static_cast<char*>(workspace) + fused_base;
        float* t[4] = {reinterpret_cast<float*>(tb), reinterpret_cast<float*>(tb + one),
                       reinterpret_cast<float*>(tb + 2 * one), reinterpret_cast<float*>(tb + 3 * one)};
        // where the passes that write "to the outputs" leave the reconstructed inputs
        float* rec = no_rec ? (np >= 2 ? reinterpret_cast<float*>(tb + 4 * one) : nullptr) : x_rec;
        float* reca = no_rec ? (np >= 2 ? reinterpret_cast<float*>(tb + 5 * one) : nullptr) : xa_rec;
        const void* cy = y; const void* cya = ya; int cy_dtype = y_dtype;
        const void* cg = dy; const void* cga = dya; int cg_dtype = dy_dtype;
        DwReducer reducer(partials, partials + (int64_t)fused_cap * wstride, wstride, s, fused_cap);
        for (size_t e = 0; e < np; ++e) {
            const FusedPass& ps = passes[np - 1 - e];
            const bool to_out = ((np - 1 - e) % 2) == 0;
            const bool last = e + 1 == np;   // writes to the outputs by construction
            float* dxr = to_out ? ((last && no_rec) ? nullptr : rec) : t[0];
            float* dxar = to_out ? ((last && no_rec) ? nullptr : reca) : t[1];
            void* ddx = to_out ? dx : static_cast<void*>(t[2]);
            void* ddxa = to_out ? dxa : static_cast<void*>(t[3]);
            const int d_dtype = to_out ? dx_dtype : NCN_F32;
            // a partial row of a multi-stage pass holds its stages side by side, as dW does
            const int rows = ps.single ? p.partial_rows : fused_grid(shape, ps, true, fused_cap) / shape->n_head;
            float* region;
            hipError_t err = reducer.reserve(rows, ps.count, &region);
            if (err != hipSuccess) return (int)err;
            if (ps.single) {
                StageArgs a{};
                fill_common(a, shape, p, first_stage + ps.first, alpha, m, activation, grouping, ps.first);
                a.in0 = cy; a.in1 = cya; a.in_dtype = cy_dtype;
                a.g0 = cg; a.g1 = cga; a.g_dtype = cg_dtype;
                a.out0 = ddx; a.out1 = ddxa; a.out_dtype = d_dtype;
                a.aux0 = dxr; a.aux1 = dxar;
                a.W = W + ps.first * wstride;
                a.dw_partials = region;
                err = run_backward_kernel(a, grouping.plain(), headwise, shape->n_head, p.grid_x, s);
                if (err == hipSuccess && grouping.ctx_len)
                    err = launch_ragged_rest(kBackward, a, shape, p.path, p.partial_rows, s);
            } else {
                FusedArgs a{};
                a.in0 = cy; a.in1 = cya; a.in_dtype = cy_dtype;
                a.g0 = cg; a.g1 = cga; a.g_dtype = cg_dtype;
                a.out0 = ddx; a.out1 = ddxa; a.out_dtype = d_dtype;
                a.aux0 = dxr; a.aux1 = dxar;
                a.W = W + ps.first * wstride;
                a.dw_partials = region;
                a.ctx_len = grouping.ctx_len;
                fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
                err = launch_fused(kBackward, a, shape, ps, s, fused_cap, headwise);
            }
            if (err != hipSuccess) return (int)err;
            reducer.add(region, rows, ps.count, dW + ps.first * wstride);
            cy = dxr; cya = dxar; cy_dtype = NCN_F32;
            cg = ddx; cga = ddxa; cg_dtype = d_dtype;
        }
        return (int)reducer.flush();
    }

    if (no_rec) {   // the state between the stages lives behind the partial rows
        if (workspace_bytes < partial_buffer_bytes(shape, row_cap) + 2 * plane_bytes) return NCN_ERR_ALIAS;
        char* cb = static_cast<char*>(workspace) + partial_buffer_bytes(shape, row_cap);
        x_rec = reinterpret_cast<float*>(cb);
        xa_rec = reinterpret_cast<float*>(cb + plane_bytes);
    }
    DwReducer reducer(partials, level1, wstride, s, row_cap);
    for (int k = n_stages - 1; k >= 0; --k) {
        float* region;
        hipError_t err = reducer.reserve(p.partial_rows + extra_rows, 1, &region);
        if (err != hipSuccess) return (int)err;
        StageArgs a{};
        fill_common(a, shape, p, first_stage + k, alpha, m, activation, grouping, k);
        const bool top = (k == n_stages - 1);
        a.in0 = top ? y : x_rec;
        a.in1 = top ? ya : xa_rec;
        a.in_dtype = top ? y_dtype : NCN_F32;
        a.g0 = top ? dy : dx;
        a.g1 = top ? dya : dxa;
        a.g_dtype = top ? dy_dtype : NCN_F32;
        a.out0 = dx;
        a.out1 = dxa;
        a.out_dtype = dx_dtype;
        a.aux0 = (no_rec && k == 0) ? nullptr : x_rec;   // the last stage to run hands nothing on
        a.aux1 = (no_rec && k == 0) ? nullptr : xa_rec;
        a.W = W + (int64_t)k * 2 * shape->E;
        a.dw_partials = region;
        err = (p.path != 2) ? launch_generic(kBackward, a, shape->n_head, p.grid_x, s)
                            : run_backward_kernel(a, grouping.plain(), headwise, shape->n_head, p.grid_x, s);
        if (err == hipSuccess && grouping.ctx_len) err = launch_ragged_rest(kBackward, a, shape, p.path, p.partial_rows, s);
        if (err != hipSuccess) return (int)err;
        reducer.add(region, p.partial_rows + extra_rows, 1, dW + k * wstride);
    }
    return (int)reducer.flush();
}

int ncn_forward(const void* x, const void* xa, int in_dtype, void* y, void* ya, int out_dtype, float* y32, float* ya32,
                const float* W, void* workspace, size_t workspace_bytes, const ncn_shape* shape, int first_stage,
                int n_stages, float alpha, float m, int activation, void* stream) {
    return forward_impl(x, xa, in_dtype, y, ya, out_dtype, y32, ya32, W, workspace, workspace_bytes,
                        Grouping{nullptr, nullptr}, shape, first_stage, n_stages, alpha, m, activation, stream);
}

int ncn_forward_indexed(const void* x, const void* xa, int in_dtype, void* y, void* ya, int out_dtype, float* y32,
                        float* ya32, const float* W, const int32_t* group_index, const int32_t* ctx_len,
                        const ncn_shape* shape, int first_stage, int n_stages, float alpha, float m, int activation,
                        void* stream) {
    return forward_impl(x, xa, in_dtype, y, ya, out_dtype, y32, ya32, W, nullptr, 0, Grouping{group_index, ctx_len},
                        shape, first_stage, n_stages, alpha, m, activation, stream);
}

int ncn_inverse(const void* y, const void* ya, int in_dtype, void* x, void* xa, int out_dtype, const float* W,
                const ncn_shape* shape, int first_stage, int n_stages, float alpha, float m, int activation,
                void* stream) {
    return inverse_impl(y, ya, in_dtype, x, xa, out_dtype, W, nullptr, 0, Grouping{nullptr, nullptr}, shape,
                        first_stage, n_stages, alpha, m, activation, stream);
}

int ncn_inverse_ws(const void* y, const void* ya, int in_dtype, void* x, void* xa, int out_dtype, const float* W,
                   void* workspace, size_t workspace_bytes, const ncn_shape* shape, int first_stage, int n_stages,
                   float alpha, float m, int activation, void* stream) {
    return inverse_impl(y, ya, in_dtype, x, xa, out_dtype, W, workspace, workspace_bytes, Grouping{nullptr, nullptr},
                        shape, first_stage, n_stages, alpha, m, activation, stream);
}

int ncn_inverse_indexed(const void* y, const void* ya, int in_dtype, void* x, void* xa, int out_dtype, const float* W,
                        const int32_t* group_index, const int32_t* ctx_len, const ncn_shape* shape, int first_stage,
                        int n_stages, float alpha, float m, int activation, void* stream) {
    return inverse_impl(y, ya, in_dtype, x, xa, out_dtype, W, nullptr, 0, Grouping{group_index, ctx_len}, shape,
                        first_stage, n_stages, alpha, m, activation, stream);
}

int ncn_backward(const void* y, const void* ya, int y_dtype, const void* dy, const void* dya, int dy_dtype, void* dx,
                 void* dxa, int dx_dtype, float* x_rec, float* xa_rec, const float* W, float* dW, void* workspace,
                 size_t workspace_bytes, const ncn_shape* shape, int first_stage, int n_stages, float alpha, float m,
                 int activation, void* stream) {
    return backward_impl(y, ya, y_dtype, dy, dya, dy_dtype, dx, dxa, dx_dtype, x_rec, xa_rec, W, dW, workspace,
                         workspace_bytes, Grouping{nullptr, nullptr}, shape, first_stage, n_stages, alpha, m, activation,
                         stream);
}

size_t ncn_static_scratch_bytes(void) { return kStaticScratchFloats * sizeof(float); }

int ncn_backward_static(const void* y, const void* ya, int y_dtype, const void* dy, const void* dya, int dy_dtype,
                        void* dx, void* dxa, int dx_dtype, float* x_rec, float* xa_rec, const float* W, float* dW,
                        const ncn_shape* shape, int first_stage, int n_stages, float alpha, float m, int activation,
                        void* stream) {
    int rc = check_shape(shape, first_stage, n_stages, activation);
    if (rc != NCN_OK) return rc;
    if (2 * shape->E > kStaticMaxTwoE) return NCN_ERR_STATIC_LIMIT;
    float* scratch = nullptr;
    const hipError_t err = static_scratch(&scratch);
    if (err != hipSuccess) return (int)err;
    return backward_impl(y, ya, y_dtype, dy, dya, dy_dtype, dx, dxa, dx_dtype, x_rec, xa_rec, W, dW, scratch,
                         partial_buffer_bytes(shape, kStaticRowCap), Grouping{nullptr, nullptr}, shape, first_stage,
                         n_stages, alpha, m, activation, stream, kStaticRowCap);
}

int ncn_backward_indexed(const void* y, const void* ya, int y_dtype, const void* dy, const void* dya, int dy_dtype,
                         void* dx, void* dxa, int dx_dtype, float* x_rec, float* xa_rec, const float* W, float* dW,
                         void* workspace, size_t workspace_bytes, const int32_t* group_index, const int32_t* ctx_len,
                         const ncn_shape* shape, int first_stage, int n_stages, float alpha, float m, int activation,
                         void* stream) {
    return backward_impl(y, ya, y_dtype, dy, dya, dy_dtype, dx, dxa, dx_dtype, x_rec, xa_rec, W, dW, workspace,
                         workspace_bytes, Grouping{group_index, ctx_len}, shape, first_stage, n_stages, alpha, m,
                         activation, stream);
}

int ncn_forward_radix(const void* x, const void* xa, int in_dtype, void* y, void* ya, int out_dtype, float* y32,
                      float* ya32, const float* W, const ncn_shape* shape, int first_level, int n_levels, float alpha,
                      float m, int activation, void* stream) {
    int rc = check_shape(shape, 0, n_levels, activation);
    if (rc != NCN_OK) return rc;
    rc = check_radix(shape, first_level, n_levels);
    if (rc != NCN_OK) return rc;
    if (!x || !xa || !y || !ya || !W) return NCN_ERR_NULL;
    if ((y32 == nullptr) != (ya32 == nullptr)) return NCN_ERR_NULL;
    if (!known_dtype(in_dtype) || !known_dtype(out_dtype)) return NCN_ERR_DTYPE;
    if (!aligned16(x) || !aligned16(xa) || !aligned16(y) || !aligned16(ya) || !aligned16(W) || !aligned16(y32) ||
        !aligned16(ya32))
        return NCN_ERR_ALIGN;
    const int path = kernel_path_for(shape, activation, alpha, m);
    if (path == 0) return NCN_ERR_UNSUPPORTED;
    ncn_shape as_wide;
    const bool headwise = headwise_call(shape, path, &as_wide);
    if (headwise) shape = &as_wide;
    const Plan p = make_plan(shape, path);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t wstride = 2 * shape->E;
    const std::vector<RadixPass> passes = plan_radix(shape, first_level, n_levels, false, path == 2);
    // every pass is closed: the first reads x, xa and the later ones run in place on y, ya; passes of several levels
    // keep their state in float32 LDS and convert on the way out
    for (size_t k = 0; k < passes.size(); ++k) {
        const RadixPass& ps = passes[k];
        const bool first = (k == 0), last = (k + 1 == passes.size());
        hipError_t err;
        if (ps.single) {
            StageArgs a{};
            Grouping g{nullptr, nullptr, first_level + ps.first};
            fill_common(a, shape, p, 0, alpha, m, activation, g, 0);
            a.in0 = first ? x : y; a.in1 = first ? xa : ya; a.in_dtype = first ? in_dtype : out_dtype;
            a.out0 = y; a.out1 = ya; a.out_dtype = out_dtype;
            a.aux0 = last ? y32 : nullptr; a.aux1 = last ? ya32 : nullptr;
            a.W = W + ps.first * wstride;
            err = (p.path != 2) ? launch_generic(kForward, a, shape->n_head, p.grid_fwd, s)
                                : run_forward_kernel(kForward, a, false, headwise, shape->n_head, p.grid_fwd, s);
        } else {
            FusedArgs a{};
            a.in0 = first ? x : y; a.in1 = first ? xa : ya; a.in_dtype = first ? in_dtype : out_dtype;
            a.out0 = y; a.out1 = ya; a.out_dtype = out_dtype;
            a.aux0 = last ? y32 : nullptr; a.aux1 = last ? ya32 : nullptr;
            a.W = W + ps.first * wstride;
            fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
            err = launch_fused_radix(kForward, a, shape, ps, s, headwise);
        }
        if (err != hipSuccess) return (int)err;
    }
    return NCN_OK;
}

int ncn_backward_radix(const void* y, const void* ya, int y_dtype, const void* dy, const void* dya, int dy_dtype,
                       void* dx, void* dxa, int dx_dtype, float* x_rec, float* xa_rec, const float* W, float* dW,
                       void* workspace, size_t workspace_bytes, const ncn_shape* shape, int first_level, int n_levels,
                       float alpha, float m, int activation, void* stream) {
    int rc = check_shape(shape, 0, n_levels, activation);
    if (rc != NCN_OK) return rc;
    rc = check_radix(shape, first_level, n_levels);
    if (rc != NCN_OK) return rc;
    if (!y || !ya || !dy || !dx || !dxa || !W || !dW) return NCN_ERR_NULL;
    if ((x_rec == nullptr) != (xa_rec == nullptr)) return NCN_ERR_NULL;
    if (!known_dtype(y_dtype) || !known_dtype(dy_dtype) || !known_dtype(dx_dtype)) return NCN_ERR_DTYPE;
    if (n_levels > 1 && dx_dtype != NCN_F32) return NCN_ERR_ALIAS;
    if (!workspace || workspace_bytes < ncn_workspace_bytes(shape)) return NCN_ERR_WORKSPACE;
    // several levels without x_rec, xa_rec: as in ncn_backward, the state travels through two arrays behind the partial
    // rows and the last pass to run writes no reconstructed inputs
    const bool no_rec = n_levels > 1 && !x_rec;
    if (no_rec) {
        const size_t plane_bytes = temp_bytes(shape, true) / 4;
        if (workspace_bytes < base_workspace_bytes(shape) + 2 * plane_bytes) return NCN_ERR_ALIAS;
        char* cb = static_cast<char*>(workspace) + base_workspace_bytes(shape);
        x_rec = reinterpret_cast<float*>(cb);
        xa_rec = reinterpret_cast<float*>(cb + plane_bytes);
    }
    if (!aligned16(y) || !aligned16(ya) || !aligned16(dy) || !aligned16(dya) || !aligned16(dx) || !aligned16(dxa) ||
        !aligned16(x_rec) || !aligned16(xa_rec) || !aligned16(W) || !aligned16(dW) || !aligned16(workspace))
        return NCN_ERR_ALIGN;
    const int path = kernel_path_for(shape, activation, alpha, m);
    if (path == 0) return NCN_ERR_UNSUPPORTED;
    ncn_shape as_wide;
    const bool headwise = headwise_call(shape, path, &as_wide);
    if (headwise) shape = &as_wide;
    const Plan p = make_plan(shape, path);
    hipStream_t s = static_cast<hipStream_t>(stream);
    float* partials = static_cast<float*>(workspace);
    float* level1 = partials + (int64_t)kMaxGridX * 2 * shape->E;
    const int64_t wstride = 2 * shape->E;
    const std::vector<RadixPass> passes = plan_radix(shape, first_level, n_levels, true, path == 2);
    // last pass first; the first one to run reads y, ya, dy, dya, the others run in place on x_rec, xa_rec, dx, dxa
    DwReducer reducer(partials, level1, wstride, s);
    for (size_t e = 0; e < passes.size(); ++e) {
        const RadixPass& ps = passes[passes.size() - 1 - e];
        const bool top = (e == 0);
        const bool drop_rec = no_rec && e + 1 == passes.size();
        const int rows = ps.single ? p.partial_rows : radix_grid(shape, ps, true) / shape->n_head;
        float* region;
        hipError_t err = reducer.reserve(rows, ps.count, &region);
        if (err != hipSuccess) return (int)err;
        if (ps.single) {
            StageArgs a{};
            Grouping g{nullptr, nullptr, first_level + ps.first};
            fill_common(a, shape, p, 0, alpha, m, activation, g, 0);
            a.in0 = top ? y : x_rec; a.in1 = top ? ya : xa_rec; a.in_dtype = top ? y_dtype : NCN_F32;
            a.g0 = top ? dy : dx; a.g1 = top ? dya : dxa; a.g_dtype = top ? dy_dtype : NCN_F32;
            a.out0 = dx; a.out1 = dxa; a.out_dtype = dx_dtype;
            a.aux0 = drop_rec ? nullptr : x_rec; a.aux1 = drop_rec ? nullptr : xa_rec;
            a.W = W + ps.first * wstride;
            a.dw_partials = region;
            err = (p.path != 2) ? launch_generic(kBackward, a, shape->n_head, p.grid_x, s)
                                : run_backward_kernel(a, false, headwise, shape->n_head, p.grid_x, s);
        } else {
            FusedArgs a{};
            a.in0 = top ? y : x_rec; a.in1 = top ? ya : xa_rec; a.in_dtype = top ? y_dtype : NCN_F32;
            a.g0 = top ? dy : dx; a.g1 = top ? dya : dxa; a.g_dtype = top ? dy_dtype : NCN_F32;
            a.out0 = dx; a.out1 = dxa; a.out_dtype = dx_dtype;
            a.aux0 = drop_rec ? nullptr : x_rec; a.aux1 = drop_rec ? nullptr : xa_rec;
            a.W = W + ps.first * wstride;
            a.dw_partials = region;
            fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
            err = launch_fused_radix(kBackward, a, shape, ps, s, headwise);
        }
        if (err != hipSuccess) return (int)err;
        reducer.add(region, rows, ps.count, dW + ps.first * wstride);
    }
    return (int)reducer.flush();
}

int ncn_inverse_radix(const void* y, const void* ya, int in_dtype, void* x, void* xa, int out_dtype, const float* W,
                      const ncn_shape* shape, int first_level, int n_levels, float alpha, float m, int activation,
                      void* stream) {
    int rc = check_shape(shape, 0, n_levels, activation);
    if (rc != NCN_OK) return rc;
    rc = check_radix(shape, first_level, n_levels);
    if (rc != NCN_OK) return rc;
    if (!x || !xa || !y || !ya || !W) return NCN_ERR_NULL;
    if (!known_dtype(in_dtype) || !known_dtype(out_dtype)) return NCN_ERR_DTYPE;
    if (!aligned16(x) || !aligned16(xa) || !aligned16(y) || !aligned16(ya) || !aligned16(W)) return NCN_ERR_ALIGN;
    const int path = kernel_path_for(shape, activation, alpha, m);
    if (path == 0) return NCN_ERR_UNSUPPORTED;
    ncn_shape as_wide;
    const bool headwise = headwise_call(shape, path, &as_wide);
    if (headwise) shape = &as_wide;
    const Plan p = make_plan(shape, path);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t wstride = 2 * shape->E;
    const std::vector<RadixPass> passes = plan_radix(shape, first_level, n_levels, false, path == 2);
    for (size_t e = 0; e < passes.size(); ++e) {   // last pass first; every pass is closed: in place after the first
        const RadixPass& ps = passes[passes.size() - 1 - e];
        const bool top = (e == 0);
        hipError_t err;
        if (ps.single) {
            StageArgs a{};
            Grouping g{nullptr, nullptr, first_level + ps.first};
            fill_common(a, shape, p, 0, alpha, m, activation, g, 0);
            a.in0 = top ? y : x; a.in1 = top ? ya : xa; a.in_dtype = top ? in_dtype : out_dtype;
            a.out0 = x; a.out1 = xa; a.out_dtype = out_dtype;
            a.W = W + ps.first * wstride;
            err = (p.path != 2) ? launch_generic(kInverse, a, shape->n_head, p.grid_fwd, s)
                                : run_forward_kernel(kInverse, a, false, headwise, shape->n_head, p.grid_fwd, s);
        } else {
            FusedArgs a{};
            a.in0 = top ? y : x; a.in1 = top ? ya : xa; a.in_dtype = top ? in_dtype : out_dtype;
            a.out0 = x; a.out1 = xa; a.out_dtype = out_dtype;
            a.W = W + ps.first * wstride;
            fill_step_table(a.tab, shape->n_cache, alpha, m, activation);
            err = launch_fused_radix(kInverse, a, shape, ps, s, headwise);
        }
        if (err != hipSuccess) return (int)err;
    }
    return NCN_OK;
}

int ncn_plan_radix(const ncn_shape* shape, int first_level, int n_levels, int activation, int backward, int32_t* out,
                   int max_passes) {
    int rc = check_shape(shape, 0, n_levels, activation);
    if (rc != NCN_OK) return rc;
    rc = check_radix(shape, first_level, n_levels);
    if (rc != NCN_OK) return rc;
    ncn_shape as_wide;
    shape = planning_shape(shape, &as_wide);
    const std::vector<RadixPass> passes = plan_radix(shape, first_level, n_levels, backward != 0);
    int k = 0;
    for (const RadixPass& p : passes) {
        if (out && k < max_passes) {
            int32_t* o = out + 6 * k;
            o[0] = p.first; o[1] = p.count; o[2] = p.single ? 0 : 1;
            o[3] = (int32_t)p.s0; o[4] = (int32_t)p.span; o[5] = (int32_t)p.rows;
        }
        ++k;
    }
    return k;
}

}  // extern "C"
