// Planning and launching of the multi-stage (LDS-resident) passes; kernels in ncn_fused_kernels.h.
#include <climits>
#include <cmath>
#include <vector>

#include "ncn_fused_dispatch.h"

namespace ncn {

namespace {

// the shapes the multi-stage kernels are built for: NCN_FOR_EACH_FUSED_CONFIG (ncn_configs.h), tile shapes as in the
// one-stage table

// One window per workgroup wherever the problem allows: workgroups that start and end on their own fall out of step
// with their neighbours on the CU, so that the loads and stores of one run under the stages of the other; a workgroup
// that loops over several windows keeps the phase it started in (measured on the 13-stage configuration: grids of
// 4096 workgroups, 4.5 windows each, 5.35 ms per step; one window each 4.94).  The backward is further bounded by its
// dW partial rows (one per n_head workgroups and stage), see fused_grid.
constexpr int kFusedMaxGridFwd = 1 << 16;
constexpr int kFusedMaxGridBwd = 1 << 16;

size_t fused_lds_bytes(int nc, int ec, bool backward, uint32_t window, int n_stages) {
    const TileShape t = fast_tile(nc, ec);
    const int lr = nc / t.r;
    // groups of two rows keep their slot-0 rows in registers (ncn_fused_pair_kernels.h): one row per group in LDS
    size_t bytes = nc == 2 ? pair_state_bytes(backward) / 2   // the arrays of the largest window, whatever this one's size
                           : (size_t)(backward ? 4 : 2) * window * nc * ec * sizeof(float);
    bytes += (size_t)kFusedMaxStages * 2 * ec * sizeof(float);  // the pass's weights
    const int nw = backward ? (nc == 2 ? kPairWavesBwd : kFusedWavesBwd) : kFusedWavesFwd;
    if (lr > 1) bytes += (size_t)nw * t.f * 64 * sizeof(float);
    if (backward) bytes += (size_t)nw * n_stages * 2 * ec * sizeof(float);
    return bytes;
}

uint32_t stage_stride_of(int stage, uint32_t groups) {
    if (stage == 0) return 0;
    uint64_t r = 1 % groups, b = 2 % groups;
    for (uint32_t e = (uint32_t)stage - 1; e; e >>= 1) {   // 2^(stage-1) mod groups by square and multiply
        if (e & 1) r = r * b % groups;
        b = b * b % groups;
    }
    return (uint32_t)r;
}

uint32_t floor_pow2(uint32_t v) {
    uint32_t p = 1;
    while (p * 2 <= v) p *= 2;
    return p;
}

}  // namespace

bool fused_supported(const ncn_shape* sh, int activation) {
    (void)activation;  // every activation has a build (tanh its own, without the branch on the code)
    const int64_t ec = sh->E / sh->n_head;
    const uint32_t groups = (uint32_t)(sh->N / sh->n_cache);
    // classes are residues modulo a power of two that divides the number of groups: an odd number of groups has none
    if (groups < 2 || (groups & 1u)) return false;
#define NCN_MATCH(NC, EC) \
    if (sh->n_cache == NC && ec == EC) return true;
    NCN_FOR_EACH_FUSED_CONFIG(NCN_MATCH)
#undef NCN_MATCH
    return false;
}

// Cuts stages [first, first + count) into passes, ascending.  Window capacity in sub-blocks is a power of two.
std::vector<FusedPass> plan_fused(const ncn_shape* sh, int first, int count, bool backward) {
    std::vector<FusedPass> passes;
    const int nc = sh->n_cache, ec = (int)(sh->E / sh->n_head);
    const uint32_t groups = (uint32_t)(sh->N / nc);
    const size_t state = nc == 2 ? pair_state_bytes(backward) : fused_state_bytes(backward);
    const uint32_t cap_rows = (uint32_t)(state / ((backward ? 4 : 2) * ec * sizeof(float)));
    uint32_t cap = floor_pow2(cap_rows / nc);
    if (cap > groups) cap = floor_pow2(groups);
    if (cap < 4) return passes;
    const uint32_t groups_pow2 = groups & (~groups + 1u);   // the power of two in the number of groups
    std::vector<uint32_t> s(count);
    for (int k = 0; k < count; ++k) s[k] = stage_stride_of(first + k, groups);

    // backward keeps a dW slot per wave and stage in LDS: 7 stages leave room for two workgroups per CU at heads of up
    // to 32 features; the two-row kernels at heads of 64 take as many stages as still let two workgroups share a CU
    // (3), at heads of 128 not even two stages would and a CU runs one workgroup of up to 7 stages
    int max_stages = backward ? kFusedMaxStages - 1 : kFusedMaxStages;
    if (backward && nc == 2) {
        const size_t budget = 80 * 1024, fixed = pair_state_bytes(true) / 2 + (size_t)kFusedMaxStages * 2 * ec * sizeof(float);
        const size_t per_stage = (size_t)kPairWavesBwd * 2 * ec * sizeof(float);
        const int fit = fixed < budget ? (int)((budget - fixed) / per_stage) : 0;
        if (fit >= 2 && fit < max_stages) max_stages = fit;
    }
    // What a pass costs, in the time one array of the activations' size takes to cross HBM at copy speed.  Traffic: the
    // pass reads `arrays_in` arrays of its windows (window / own times the data) and writes `arrays_out` arrays of its
    // owned rows; in the backward the pass that holds the call's first stage runs last and writes the two gradients
    // only (callers that want the reconstructed inputs pay two arrays more than priced here).  Issue: every stage costs
    // `per_stage` such units of instruction issue on all groups of its windows (measured per kernel family on
    // x[128, 8192, 128]: a two-row backward stage 0.143 ms against 0.102 ms per array, a two-row forward stage 0.078 ms;
    // the four-row kernels in proportion to their instruction counts).  The two overlap, better the more they differ:
    // the cube root of the sum of cubes follows the measured pass times to 5 % (a closed backward pass, whose windows
    // are the most scattered in memory, takes 1.1 times that).
    const double arrays_in = backward ? 4.0 : 2.0;
    const double per_stage = nc == 2 ? (backward ? 1.4 : 0.76) : (backward ? 3.6 : 2.0);
    auto priced = [&](int a, double redundancy, int stages, bool closed) -> double {
        const double arrays_out = backward ? (a == 0 ? 2.0 : 4.0) : 2.0;
        const double traffic = arrays_in * redundancy + arrays_out;
        const double issue = per_stage * stages * redundancy;
        return std::cbrt(traffic * traffic * traffic + issue * issue * issue) * (closed && backward ? 1.1 : 1.0);
    };
    // stages [a, b) as one pass; returns its cost (see above), or < 0 if impossible
    auto make = [&](int a, int b, FusedPass& p) -> double {
        if (b - a > max_stages || b - a < 2) return -1.0;
        // S0: the largest power of two that divides every non-zero stride of the pass and the number of groups (with a
        // power of two of groups the strides are powers of two and this is the smallest of them; with 3 * 2^k groups
        // and the like the strides past 2^k wrap to odd multiples of 2^k)
        uint32_t s0 = 0;
        for (int k = a; k < b; ++k)
            if (s[k]) {
                const uint32_t low = s[k] & (~s[k] + 1u);
                if (!s0 || low < s0) s0 = low;
            }
        if (s0 > groups_pow2) s0 = groups_pow2;
        if (!s0) {  // only contiguous-block stages: any class structure works, take full windows
            s0 = groups_pow2;
            while (s0 > 1 && groups / s0 < cap) s0 /= 2;
        }
        p.first = a;
        p.count = b - a;
        p.single = 0;
        p.class_stride = s0;
        p.ring = groups / s0;
        uint32_t sum = 0;
        for (int k = a; k < b; ++k) {
            if (s[k] % s0) return -1.0;
            p.sub_stride[k - a] = s[k] / s0;
            sum += s[k] / s0;
        }
        if (p.ring <= cap_rows / nc) {  // closed: whole rings of adjacent classes, a power of two of them per window
            uint32_t rings = floor_pow2((cap_rows / nc) / p.ring);
            if (rings > s0) rings = s0;
            p.closed = 1;
            p.window = rings * p.ring;
            p.halo = 0;
            p.own = p.window;
            p.tiles_per_ring = 1;
            p.class_groups = s0 / rings;
            return priced(a, 1.0, b - a, true);
        }
        p.closed = 0;
        p.window = cap;
        p.halo = (uint32_t)(nc - 1) * sum;
        if (2 * p.halo >= cap) return -1.0;
        p.own = cap - 2 * p.halo;
        if (p.own * 4 < cap * 3) return -1.0;  // more than a third of the window would be redundant work
        p.tiles_per_ring = (p.ring + p.own - 1) / p.own;
        p.class_groups = s0;
        return priced(a, (double)cap / p.own, b - a, false);
    };

    // cheapest cut of the range into passes (a one-stage launch is bound by its traffic: every array once)
    std::vector<double> best(count + 1, 1e30);
    std::vector<int> from(count + 1, -1);
    std::vector<FusedPass> how(count + 1);
    best[0] = 0.0;
    for (int b = 1; b <= count; ++b) {
        const double single = arrays_in + (backward ? (b == 1 ? 2.0 : 4.0) : 2.0);
        if (best[b - 1] + single < best[b]) {
            best[b] = best[b - 1] + single;
            from[b] = b - 1;
            FusedPass p{};
            p.first = b - 1;
            p.count = 1;
            p.single = 1;
            how[b] = p;
        }
        for (int a = b - 2; a >= 0 && b - a <= max_stages; --a) {
            FusedPass p{};
            const double c = make(a, b, p);
            if (c >= 0.0 && best[a] + c < best[b] - 1e-9) {
                best[b] = best[a] + c;
                from[b] = a;
                how[b] = p;
            }
        }
    }
    for (int b = count; b > 0; b = from[b]) passes.insert(passes.begin(), how[b]);
    return passes;
}

int64_t fused_items(const ncn_shape* sh, const FusedPass& p) {
    return sh->batch * (int64_t)p.class_groups * p.tiles_per_ring * sh->n_head;
}

int fused_grid(const ncn_shape* sh, const FusedPass& p, bool backward, int row_cap) {
    const int64_t items = fused_items(sh, p);
    // the forward kernels for groups of two rows take one window per workgroup and nothing else
    if (!backward && sh->n_cache == 2) return items <= INT_MAX ? (int)items : 0;
    int64_t cap = backward ? kFusedMaxGridBwd : kFusedMaxGridFwd;
    if (backward) {  // partial rows (grid / n_head) * stages must fit the row_cap rows of the dW scratch
        const int64_t by_rows = (int64_t)row_cap / p.count * sh->n_head;
        if (by_rows < cap) cap = by_rows;
    }
    int64_t g = items < cap ? items : cap;
    g = g / sh->n_head * sh->n_head;
    if (g < sh->n_head) g = sh->n_head;
    return (int)g;
}

hipError_t launch_fused(Pass pass, FusedArgs& a, const ncn_shape* sh, const FusedPass& p, hipStream_t s, int row_cap,
                        bool headwise) {
    const bool backward = pass == kBackward;
    const int nc = sh->n_cache, ec = (int)(sh->E / sh->n_head);
    a.N = sh->N;
    a.E = sh->E;
    a.n_head = sh->n_head;
    a.n_stages = p.count;
    a.class_stride = p.class_stride;
    a.ring = p.ring;
    a.ring_magic = (p.ring & (p.ring - 1)) == 0 ? 0u : (uint32_t)(((1ull << 32) + p.ring - 1) / p.ring);
    a.window = p.window;
    a.halo = p.halo;
    a.own = p.own;
    a.tiles_per_ring = p.tiles_per_ring;
    a.closed = p.closed;
    a.class_groups = p.class_groups;
    a.total_items = (uint32_t)fused_items(sh, p);
    for (int k = 0; k < kFusedMaxStages; ++k) a.sub_stride[k] = k < p.count ? p.sub_stride[k] : 0;
    a.scale_dn = (float)std::pow((double)a.tab.m, (double)(nc * p.count));
    a.scale_up = (float)std::pow((double)a.tab.m, -(double)(nc * p.count));
    const int grid = fused_grid(sh, p, backward, row_cap);
    const size_t lds = fused_lds_bytes(nc, ec, backward, p.window, p.count);
    if (headwise) return launch_fused_headwise(pass, a, nc, ec, grid, lds, s);
    if (a.ctx_len) return launch_fused_lengths(pass, a, nc, ec, grid, lds, s);
    return launch_fused_shape<false, false, false>(pass, a, nc, ec, grid, lds, s);
}

}  // namespace ncn
