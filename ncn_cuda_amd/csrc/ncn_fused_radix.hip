// Planning and launching of multi-stage passes over levels of the radix-n digit grouping
// (ncn_triton/group_tensors.py:8-18); the kernels are the RADIX builds of ncn_fused_kernels.h.
#include <cmath>
#include <vector>

#include "ncn_fused_dispatch.h"

namespace ncn {

namespace {

// shapes with a radix build: digits are extracted with shifts, so n_cache is 2 or 4 (tile shapes of the one-stage table)
#define NCN_FOR_EACH_RADIX_CONFIG(X) NCN_FOR_EACH_FUSED_CONFIG(X)

constexpr int kRadixMaxGrid = 4096;

uint32_t floor_pow2(uint32_t v) {
    uint32_t p = 1;
    while (p * 2 <= v) p *= 2;
    return p;
}

size_t radix_lds_bytes(int nc, int ec, bool backward, uint32_t rows, int n_stages) {
    const TileShape t = fast_tile(nc, ec);
    const int lr = nc / t.r;
    size_t bytes = (size_t)(backward ? 4 : 2) * rows * ec * sizeof(float);
    bytes += (size_t)kFusedMaxStages * 2 * ec * sizeof(float);
    const int nw = backward ? kFusedWavesBwd : kFusedWavesFwd;
    if (lr > 1) bytes += (size_t)nw * t.f * 64 * sizeof(float);
    if (backward) bytes += (size_t)nw * n_stages * 2 * ec * sizeof(float);
    return bytes;
}

int64_t ipow(int64_t b, int e) {
    int64_t r = 1;
    for (int k = 0; k < e; ++k) r *= b;
    return r;
}

}  // namespace

bool radix_fused_supported(const ncn_shape* sh) {
    const int64_t ec = sh->E / sh->n_head;
#define NCN_MATCH(NC, EC) \
    if (sh->n_cache == NC && ec == EC) return true;
    NCN_FOR_EACH_RADIX_CONFIG(NCN_MATCH)
#undef NCN_MATCH
    return false;
}

// Levels [first, first + count) cut into passes of as many levels as fit the LDS budget (and the stage limits of the
// kernels); a pass of one level is left to the one-stage kernel.  Every pass is closed.
std::vector<RadixPass> plan_radix(const ncn_shape* sh, int first, int count, bool backward, bool fused) {
    std::vector<RadixPass> passes;
    const int nc = sh->n_cache, ec = (int)(sh->E / sh->n_head);
    const uint32_t cap_rows = floor_pow2((uint32_t)(fused_state_bytes(backward) / ((backward ? 4 : 2) * ec * sizeof(float))));
    int kmax = 0;
    while (ipow(nc, kmax + 1) <= (int64_t)cap_rows) ++kmax;
    const int max_stages = backward ? kFusedMaxStages - 1 : kFusedMaxStages;
    if (kmax > max_stages) kmax = max_stages;
    for (int a = 0; a < count;) {
        RadixPass p{};
        p.first = a;
        p.count = (count - a < kmax) ? count - a : kmax;
        p.single = (p.count < 2 || !fused || !radix_fused_supported(sh)) ? 1 : 0;
        if (p.single) p.count = 1;
        p.s0 = (uint32_t)ipow(nc, first + a);
        p.span = (uint32_t)ipow(nc, p.count);
        // A workgroup holds a whole number of windows, and every workgroup-load of a batch entry holds the same
        // number: the largest divisor of the window count that the LDS budget takes (N = odd * n^k leaves an odd
        // factor in the window count; a count that does not divide would leave the last windows unprocessed).
        const uint32_t windows = (uint32_t)(sh->N / p.span);   // per batch entry and head
        uint32_t per_load = cap_rows / p.span;
        if (per_load > windows) per_load = windows;            // N smaller than the LDS budget
        while (windows % per_load) --per_load;
        p.rows = per_load * p.span;
        p.loads = windows / per_load;
        passes.push_back(p);
        a += p.count;
    }
    return passes;
}

int radix_grid(const ncn_shape* sh, const RadixPass& p, bool backward) {
    const int64_t items = sh->batch * (int64_t)p.loads * sh->n_head;
    int64_t cap = kRadixMaxGrid;
    if (backward) {
        const int64_t by_rows = (int64_t)kMaxGridX / p.count * sh->n_head;
        if (by_rows < cap) cap = by_rows;
    }
    int64_t g = items < cap ? items : cap;
    g = g / sh->n_head * sh->n_head;
    if (g < sh->n_head) g = sh->n_head;
    return (int)g;
}

hipError_t launch_fused_radix(Pass pass, FusedArgs& a, const ncn_shape* sh, const RadixPass& p, hipStream_t s,
                              bool headwise) {
    const bool backward = pass == kBackward;
    const int nc = sh->n_cache, ec = (int)(sh->E / sh->n_head);
    a.N = sh->N;
    a.E = sh->E;
    a.n_head = sh->n_head;
    a.n_stages = p.count;
    a.class_stride = p.s0;
    a.ring = p.span;
    a.window = p.rows / nc;
    a.halo = 0;
    a.own = a.window;
    a.tiles_per_ring = 1;
    a.closed = 1;
    a.class_groups = p.loads;
    a.total_items = (uint32_t)(sh->batch * (int64_t)p.loads * sh->n_head);
    for (int k = 0; k < kFusedMaxStages; ++k) a.sub_stride[k] = k < p.count ? (uint32_t)ipow(nc, k) : 0;
    a.scale_dn = (float)std::pow((double)a.tab.m, (double)(nc * p.count));
    a.scale_up = (float)std::pow((double)a.tab.m, -(double)(nc * p.count));
    const int grid = radix_grid(sh, p, backward);
    const size_t lds = radix_lds_bytes(nc, ec, backward, p.rows, p.count);
    if (headwise) return launch_fused_radix_headwise(pass, a, nc, ec, grid, lds, s);
    return launch_fused_shape<true, false, false>(pass, a, nc, ec, grid, lds, s);
}

}  // namespace ncn
