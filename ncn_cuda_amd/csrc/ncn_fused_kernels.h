// Multi-stage kernels: several consecutive stages on a tile of rows that stays in LDS.
//
// Why.  With small groups (n_cache 2..8) one stage does little arithmetic per byte and a one-stage launch runs
// at HBM speed; every further stage that works on rows already in LDS saves one full read and write of the
// activations (and, in backward, of the gradients).
//
// Which rows.  Stage l reads, for group b, slot o from block (b + o*s_l) mod groups (torch_ref/ncn_pytorch.py:38-40).
// Take a run of stages whose non-zero strides are all multiples of S0 (powers of two here).  Then blocks of one
// residue class r = b mod S0 only ever meet blocks of the same class, and inside a class, with the sub-block
// index q = b div S0 on a ring of groups/S0 sub-blocks, the strides become s_l/S0.  A workgroup holds a window
// of consecutive sub-blocks of one (batch, head, class):
//   * closed pass: the window is one whole ring, or several whole rings of adjacent classes when a ring is
//     smaller than the window (indices wrap inside each ring): nothing outside is ever needed;
//   * halo pass:   the window is `own` sub-blocks plus `halo` = (n_cache-1) * sum(s_l/S0) on each side.  Every
//     stage updates the groups that lie completely inside the window; rows near the window edge go stale, but
//     by construction never reach an owned row.  Only owned rows are written back and only groups whose slot-0
//     sub-block is owned count towards dW, so the redundant halo work is invisible outside.
// A halo pass must not run in place (another workgroup still needs the old value of an owned row as its halo),
// a closed pass may.  The host (ncn_fused.hip) cuts a stage range into passes and ping-pongs buffers.
//
// How.  Per stage each wave gathers R x F register tiles of whole groups from LDS (the tile shapes and the step
// code are those of the one-stage kernels, ncn_stage_kernels.h), runs the n_cache steps and scatters the tile
// back; one workgroup barrier separates stages.  The rows stay in the scaled form of the step code for the whole pass
// (xs and as or bh, see StepTable; backward keeps G = g / m^t and P = p / m^t with the step counter counting across
// the stages, p = (1-m) g + h in place of h), so true values exist only in HBM.  The pass's weights sit in LDS,
// already scaled by gamma.  Backward sums each wave's dW share of a stage into a per-wave LDS
// slot (one writer per slot, fixed order: deterministic) and leaves one partial row per workgroup and stage.
//
// RADIX builds of the same kernels run levels of the radix-n digit grouping (ncn_triton/group_tensors.py:8-18)
// instead: level l groups the n_cache positions that differ only in base-n_cache digit l.  A run of levels a .. a+k-1
// only ever mixes the positions lower + n^a * d + n^(a+k) * upper, d = 0 .. n^k - 1, of one (lower, upper): a closed
// window of n^k rows, no halo at all, any pass may run in place.  A workgroup holds rows / n^k such windows; the LDS
// row of digit string d is d itself, and level a+j pairs the rows whose d differ in digit j.  (n_cache 2 and 4
// only: every size below is a power of two and the digit arithmetic is shifts.)
#pragma once
#include "ncn_headwise_kernels.h"

namespace ncn {

// The step code is instantiated with ROWS = true here: these kernels wait on latency rather than on issue slots, and
// reductions through DPP row operations come back sooner than through the LDS crossbar (measured 2.5 % on 13 stages).
constexpr int kFusedMaxStages = 8;
// LDS for the row arrays of one workgroup (2 forward and inverse, 4 backward)
#ifndef NCN_FUSED_STATE_FWD
#define NCN_FUSED_STATE_FWD (64 * 1024)
#endif
constexpr size_t kFusedStateBytesFwd = NCN_FUSED_STATE_FWD;
constexpr size_t kFusedStateBytesBwd = 64 * 1024;
constexpr size_t fused_state_bytes(bool backward) { return backward ? kFusedStateBytesBwd : kFusedStateBytesFwd; }
// Groups of two rows under the stride permutation keep half of a window in registers (ncn_fused_pair_kernels.h): the
// bytes of both halves that one workgroup holds
#ifndef NCN_PAIR_STATE_FWD
#define NCN_PAIR_STATE_FWD (128 * 1024)
#endif
#ifndef NCN_PAIR_STATE_BWD
#define NCN_PAIR_STATE_BWD (128 * 1024)
#endif
constexpr size_t kPairStateBytesFwd = NCN_PAIR_STATE_FWD, kPairStateBytesBwd = NCN_PAIR_STATE_BWD;
constexpr size_t pair_state_bytes(bool backward) { return backward ? kPairStateBytesBwd : kPairStateBytesFwd; }
#ifndef NCN_FUSED_WAVES_FWD
#define NCN_FUSED_WAVES_FWD 8
#endif
constexpr int kFusedWavesFwd = NCN_FUSED_WAVES_FWD;   // (16 waves per workgroup measured slower: all waves of a workgroup share its phases)
constexpr int kFusedWavesBwd = 8;   // backward runs at 128 VGPRs: 4 waves per SIMD in all

struct FusedArgs {
    const void* in0;   // forward: x    backward: y (outputs of the pass's last stage)
    const void* in1;   //          xa             ya
    const void* g0;    // backward: dy
    const void* g1;    //           dya (may be null = zeros)
    void* out0;        // forward: y    backward: dx
    void* out1;        //          ya             dxa
    float* aux0;       // forward: optional float32 copy of y     backward: x_rec (inputs of the pass's first stage)
    float* aux1;       //          optional float32 copy of ya              xa_rec
    const float* W;    // [n_stages][2E], first stage of the pass first
    float* dw_partials;  // backward: [gridDim.x / n_head][n_stages][2E]
    const int32_t* ctx_len;  // LENGTHS builds: [batch] live slots per batch entry (in the group order of each stage)
    int64_t N, E;
    int32_t n_head, n_stages;
    int32_t in_dtype, g_dtype, out_dtype;
    uint32_t ring_magic;      // 0 when `ring` is a power of two, else ceil(2^32 / ring): closed passes divide by the ring
    // RADIX builds read: class_stride = n^a in rows, ring = n^k rows per window, window = rows / n_cache,
    // class_groups = workgroup-loads per batch entry, sub_stride[j] = n^j in rows, closed = 1
    uint32_t class_stride;    // S0, in blocks
    uint32_t ring;            // sub-blocks per class = groups / S0 (a power of two, or an odd number times one)
    uint32_t window;          // sub-blocks held in LDS
    uint32_t halo;            // sub-blocks of halo on each side (0 for a closed pass)
    uint32_t own;             // owned sub-blocks per window (= ring for a closed pass)
    uint32_t tiles_per_ring;  // ceil(ring / own)
    uint32_t closed;          // 1: the window holds window/ring whole rings (adjacent classes) and indices wrap
    uint32_t class_groups;    // closed: S0 / (window / ring) windows per batch entry; halo: S0
    uint32_t total_items;     // batch * class_groups * tiles_per_ring * n_head
    uint32_t sub_stride[kFusedMaxStages];  // s_l / S0 per stage of the pass
    float scale_dn, scale_up;              // m^(n_cache * n_stages) and its reciprocal (backward: gradients leave as G m^T)
    StepTable tab;
};

struct FusedItem {
    int head;
    uint32_t cls, sub0, own_lo, own_cnt, batch;
    int64_t base;  // element offset of (batch, row 0, head slice)
};

__device__ __forceinline__ uint32_t log2u(uint32_t v) { return 31u - (uint32_t)__clz((int)v); }

// Closed passes hold whole rings side by side in a window: number of the ring that window position q lies in
// (q < 2^16: a window has at most a few thousand positions, which keeps the multiply-high exact).
__device__ __forceinline__ uint32_t ring_index(const FusedArgs& A, uint32_t q) {
    return A.ring_magic == 0u ? q >> log2u(A.ring) : __umulhi(q, A.ring_magic);
}
// Window position of the sub-block `add` places after q on q's own ring (closed passes; add < 4 * ring).
__device__ __forceinline__ uint32_t ring_wrap(const FusedArgs& A, uint32_t q, uint32_t add) {
    if (A.ring_magic == 0u) return (q & ~(A.ring - 1u)) | ((q + add) & (A.ring - 1u));
    // rings of 3 * 2^k and the like.  The ring's first position does not change from stage to stage, but it is made
    // afresh each time (the empty statement hides q from the optimiser): kept in a register across the stages of a
    // pass it would cost the kernels that run at their register limit a spill.
    uint32_t qq = q;
    asm volatile("" : "+v"(qq));
    const uint32_t base = __umulhi(qq, A.ring_magic) * A.ring;
    uint32_t t = qq - base + add;
    t -= __umulhi(t, A.ring_magic) * A.ring;
    return base + t;
}
// (sub-block on the ring, class) of window position qi
__device__ __forceinline__ void ring_place(const FusedArgs& A, uint32_t sub0, uint32_t cls0, uint32_t qi, uint32_t& sub,
                                           uint32_t& cls) {
    if (A.closed) {       // whole rings of adjacent classes, the first sub-block of each first
        const uint32_t ri = ring_index(A, qi);
        sub = qi - ri * A.ring;
        cls = cls0 + ri;
    } else {              // a stretch of one ring, shorter than the ring: wraps at most once
        sub = sub0 + qi;
        if (sub >= A.ring) sub -= A.ring;
        cls = cls0;
    }
}

template <int NC, int EC, bool RADIX>
__device__ __forceinline__ FusedItem fused_item(const FusedArgs& A, uint32_t item) {
    FusedItem it;
    it.head = item % A.n_head;
    uint32_t t = item / A.n_head;
    const uint32_t k = t % A.tiles_per_ring;
    t /= A.tiles_per_ring;
    const uint32_t cg = t % A.class_groups;
    const uint32_t b = t / A.class_groups;
    if (RADIX) {
        it.cls = cg * (A.window * NC / A.ring);   // number of the first window: (upper, lower) = (u / n^a, u % n^a)
        it.sub0 = 0u;
        it.own_lo = 0u;
        it.own_cnt = A.window;
    } else if (A.closed) {
        it.cls = cg * (A.window / A.ring);   // first class of the window
        it.sub0 = 0u;
        it.own_lo = 0u;
        it.own_cnt = A.window;
    } else {
        it.cls = cg;
        it.sub0 = k * A.own + A.ring - A.halo;   // k * own < ring
        if (it.sub0 >= A.ring) it.sub0 -= A.ring;
        it.own_lo = A.halo;
        const uint32_t left = A.ring - k * A.own;
        it.own_cnt = left < A.own ? left : A.own;
    }
    it.batch = b;
    it.base = (int64_t)b * A.N * A.E + (int64_t)it.head * EC;
    return it;
}

// element offset (without the feature) of local row `lr` = (window sub-block qi) * NC + slot
template <int NC, bool RADIX>
__device__ __forceinline__ int64_t fused_row_offset(const FusedArgs& A, const FusedItem& it, uint32_t lr) {
    if (RADIX) {
        const uint32_t lg_span = log2u(A.ring), lg_s0 = log2u(A.class_stride);
        const uint32_t d = lr & (A.ring - 1u), u = it.cls + (lr >> lg_span);
        const int64_t pos = (int64_t)(u & (A.class_stride - 1u)) + ((int64_t)d << lg_s0) +
                            ((int64_t)(u >> lg_s0) << (lg_s0 + lg_span));
        return it.base + pos * A.E;
    }
    const uint32_t qi = lr / NC, o = lr - qi * NC;
    uint32_t sub, cls;
    ring_place(A, it.sub0, it.cls, qi, sub, cls);
    const uint32_t blk = sub * A.class_stride + cls;
    return it.base + ((int64_t)blk * NC + o) * A.E;
}

// Where window row `lr` lies in LDS.  The rows of one slot of neighbouring groups are NC rows apart, i.e. a multiple of
// 256 bytes at these head widths: they would all start in the same LDS bank.  Flipping the row's lowest bit with the
// bit above its slot number puts every other one of them half the banks further (rows stay whole, pairs swap places).
template <int NC>
__device__ __forceinline__ uint32_t fused_lds_place(uint32_t lr) {
    constexpr uint32_t lg = NC == 2 ? 1u : NC == 4 ? 2u : 3u;
    return lr ^ ((lr >> lg) & 1u);
}

// LDS row of slot i of the group whose slot-0 sub-block is window position qg
// (RADIX: row of digit i at level log_n(sstride) of group qg; groups are numbered window by window)
template <int NC, bool RADIX>
__device__ __forceinline__ uint32_t fused_lds_row(const FusedArgs& A, uint32_t qg, uint32_t i, uint32_t sstride) {
    if (RADIX) {
        constexpr uint32_t lg_nc = NC == 2 ? 1u : 2u;
        static_assert(NC == 2 || NC == 4, "digit arithmetic by shifts");
        const uint32_t lg_span = log2u(A.ring), lg_sj = log2u(sstride);
        const uint32_t gpw = A.ring >> lg_nc;                       // groups per window
        const uint32_t wq = qg >> (lg_span - lg_nc), g = qg & (gpw - 1u);
        return fused_lds_place<NC>((wq << lg_span) + ((g >> lg_sj) << (lg_sj + lg_nc)) + (i << lg_sj) + (g & (sstride - 1u)));
    }
    const uint32_t qi = A.closed ? ring_wrap(A, qg, i * sstride) : qg + i * sstride;  // closed: inside the group's own ring
    return fused_lds_place<NC>(qi * NC + i);
}

// Live rows of the group whose slot-0 sub-block is window position qg, for a batch entry with `len` live slots: the
// group's number is the block of its slot 0 (the stride permutation leaves slot 0 in place), its slots are
// number * NC + 0 .. NC-1 (ncn_triton/ncn_triton_old.py:66, 93-96).
template <int NC>
__device__ __forceinline__ int fused_live_rows(const FusedArgs& A, const FusedItem& it, uint32_t qg, int32_t len) {
    uint32_t sub, cls;
    ring_place(A, it.sub0, it.cls, qg, sub, cls);
    const int64_t r = (int64_t)len - (int64_t)(sub * A.class_stride + cls) * NC;
    return (int)max((int64_t)0, min(r, (int64_t)NC));
}

template <int F>
__device__ __forceinline__ void lds_load_frag(const float* row, float (&v)[F]) {
#pragma unroll
    for (int k = 0; k < F / 4; ++k) {
        const float4 t = reinterpret_cast<const float4*>(row)[k];
        v[4 * k] = t.x; v[4 * k + 1] = t.y; v[4 * k + 2] = t.z; v[4 * k + 3] = t.w;
    }
}
template <int F>
__device__ __forceinline__ void lds_store_frag(float* row, const float (&v)[F]) {
#pragma unroll
    for (int k = 0; k < F / 4; ++k)
        reinterpret_cast<float4*>(row)[k] = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
}

// Window rows on their way from global memory to LDS: 4 features per thread and trip, kept as raw bits so that
// nothing waits for the loads until fused_commit_rows turns them into floats.  A workgroup fetches the window of
// its next item while it computes the current one.
template <int NC, int EC, int NW, int K, bool RADIX>
__device__ __forceinline__ void fused_window_offsets(const FusedArgs& A, const FusedItem& it, uint32_t rows,
                                                     int64_t (&off)[K]) {
    constexpr uint32_t CPR = EC / 4;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        // a trip past the end re-reads the last chunk, which fused_commit_rows ignores
        const uint32_t c = min(threadIdx.x + k * 64 * NW, rows * CPR - 1u);
        const uint32_t lr = c / CPR, c4 = c - lr * CPR;
        off[k] = fused_row_offset<NC, RADIX>(A, it, lr) + c4 * 4;
    }
}

// one wave-uniform branch around straight runs of loads: nothing between the loads makes one wait for another
template <int K>
__device__ __forceinline__ void fused_fetch_rows(const void* src, int dtype, const int64_t (&off)[K], uint4 (&raw)[K]) {
    if (!src) {
#pragma unroll
        for (int k = 0; k < K; ++k) raw[k] = make_uint4(0u, 0u, 0u, 0u);
    } else if (dtype == NCN_F32) {
#pragma unroll
        for (int k = 0; k < K; ++k) raw[k] = *reinterpret_cast<const uint4*>(static_cast<const float*>(src) + off[k]);
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint2 t = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(src) + off[k]);
            raw[k] = make_uint4(t.x, t.y, 0u, 0u);
        }
    }
}

__device__ __forceinline__ void fused_raw_to_float(const uint4& r, int dtype, float (&v)[4]) {
    if (dtype == NCN_F32) {
        v[0] = __uint_as_float(r.x); v[1] = __uint_as_float(r.y); v[2] = __uint_as_float(r.z); v[3] = __uint_as_float(r.w);
    } else {
        v[0] = bf16_to_f32(r.x & 0xffffu); v[1] = bf16_to_f32(r.x >> 16);
        v[2] = bf16_to_f32(r.y & 0xffffu); v[3] = bf16_to_f32(r.y >> 16);
    }
}

template <int NC, int EC, int NW, int K>
__device__ __forceinline__ void fused_commit_rows(const uint4 (&raw)[K], int dtype, float* dst, uint32_t rows, float scale) {
    constexpr uint32_t CPR = EC / 4;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = threadIdx.x + k * 64 * NW;
        if (c < rows * CPR) {
            float v[4];
            fused_raw_to_float(raw[k], dtype, v);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] *= scale;
            lds_store_frag<4>(dst + fused_lds_place<NC>(c / CPR) * EC + (c % CPR) * 4, v);
        }
    }
}

// LDS -> global for the owned rows, each value times `scale`
template <int NC, int EC, int NW, bool RADIX>
__device__ __forceinline__ void fused_store_rows_scaled(const FusedArgs& A, const FusedItem& it, const float* src,
                                                        float scale, void* dst, int dtype, float* copy32) {
    constexpr uint32_t CPR = EC / 4;
    const uint32_t r0 = it.own_lo * NC, rows = it.own_cnt * NC;
    for (uint32_t c = threadIdx.x; c < rows * CPR; c += 64 * NW) {
        const uint32_t lr = r0 + c / CPR, c4 = c % CPR;
        float v[4];
        lds_load_frag<4>(src + fused_lds_place<NC>(lr) * EC + c4 * 4, v);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] *= scale;
        const int64_t off = fused_row_offset<NC, RADIX>(A, it, lr) + c4 * 4;
        store_frag<4>(dst, dtype, off, true, v);
        if (copy32) store_frag<4>(copy32, NCN_F32, off, true, v);
    }
}

// the pass's weights times gamma, [stage][Wi | Wj][EC] of this workgroup's head, into LDS
template <int EC, int NW>
__device__ __forceinline__ void fused_load_weights(const FusedArgs& A, int head, float* w_lds) {
    for (int k = threadIdx.x; k < A.n_stages * 2 * EC; k += 64 * NW) {
        const int st = k / (2 * EC), rem = k - st * 2 * EC, half = rem / EC, f = rem - half * EC;
        w_lds[k] = A.tab.gamma * A.W[(int64_t)st * 2 * A.E + (int64_t)half * A.E + (int64_t)head * EC + f];
    }
}

// TANH_ONLY as in the one-stage kernels: the tanh build has no branch on the activation code.
// INVERSE: the same kernel undoes the stages instead, last one first (in0, in1 = y, ya; out0, out1 = x, xa).
// LENGTHS: one context length per batch entry; the group a length cuts runs its live steps on its live rows, rows
// past the length stay in LDS as they came (a row may be live in one stage of the pass and past the length in another).
// HEADWISE: heads of one feature laid out as heads of EC adjacent ones (ncn_headwise_kernels.h): the same windows, tiles
// and weights, the step code without sums across a row's lanes.
template <int NC, int EC, int R, int F, bool TANH_ONLY, bool RADIX = false, bool INVERSE = false, bool LENGTHS = false,
          bool HEADWISE = false>
__global__ void __launch_bounds__(64 * kFusedWavesFwd) fused_forward_kernel(const FusedArgs A) {
    static_assert(!(RADIX && LENGTHS), "context lengths go with the stride permutation");
    constexpr int NW = kFusedWavesFwd;
    using T = Tile<NC, EC, R, F>;
    extern __shared__ float4 fused_lds4[];
    float* lds = reinterpret_cast<float*>(fused_lds4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fl = lane % T::LF, rl = (lane / T::LF) % T::LR, gw = lane / T::LPG;
    const uint32_t rows = A.window * NC;
    float* xs = lds;
    float* as = lds + rows * EC;
    float* w_lds = as + rows * EC;                              // [kFusedMaxStages][2][EC]
    float4* slots = reinterpret_cast<float4*>(w_lds + kFusedMaxStages * 2 * EC) + wave * (F / 4) * 64;
    fused_load_weights<EC, NW>(A, blockIdx.x % A.n_head, w_lds);   // every item of this workgroup has this head

    // trips of 64 * NW threads over the float4 chunks of the largest window the LDS budget allows
    constexpr int K = (int)((kFusedStateBytesFwd / 2 / sizeof(float4) + 64 * NW - 1) / (64 * NW));
    uint4 rx[K], ra[K];
    if (blockIdx.x < A.total_items) {
        int64_t off[K];
        fused_window_offsets<NC, EC, NW, K, RADIX>(A, fused_item<NC, EC, RADIX>(A, blockIdx.x), rows, off);
        fused_fetch_rows<K>(A.in0, A.in_dtype, off, rx);
        fused_fetch_rows<K>(A.in1, A.in_dtype, off, ra);
    }
    for (uint32_t item = blockIdx.x; item < A.total_items; item += gridDim.x) {
        const FusedItem it = fused_item<NC, EC, RADIX>(A, item);
        const int32_t len = LENGTHS ? max(0, min(A.ctx_len[it.batch], (int32_t)A.N)) : 0;
        fused_commit_rows<NC, EC, NW, K>(rx, A.in_dtype, xs, rows, A.tab.kappa);
        fused_commit_rows<NC, EC, NW, K>(ra, A.in_dtype, as, rows, INVERSE ? A.tab.b_scale : A.tab.a_scale);
        __syncthreads();
        if (item + gridDim.x < A.total_items) {   // the next window travels while this one is computed
            int64_t off[K];
            fused_window_offsets<NC, EC, NW, K, RADIX>(A, fused_item<NC, EC, RADIX>(A, item + gridDim.x), rows, off);
            fused_fetch_rows<K>(A.in0, A.in_dtype, off, rx);
            fused_fetch_rows<K>(A.in1, A.in_dtype, off, ra);
        }
        for (int sq = 0; sq < A.n_stages; ++sq) {
            const int st = INVERSE ? A.n_stages - 1 - sq : sq;
            const uint32_t ss = A.sub_stride[st];
            const uint32_t ngroups = A.closed ? A.window : A.window - (NC - 1) * ss;
            float wi[F], wj[F];
            lds_load_frag<F>(w_lds + st * 2 * EC + fl * F, wi);
            lds_load_frag<F>(w_lds + st * 2 * EC + EC + fl * F, wj);
            for (uint32_t wt = wave; wt * T::GPW < ngroups; wt += NW) {
                const uint32_t qg = wt * T::GPW + gw;
                const bool valid = qg < ngroups;
                float x[R][F], a[R][F];
                uint32_t row[R];
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    row[rr] = fused_lds_row<NC, RADIX>(A, valid ? qg : 0u, rl * R + rr, ss) * EC + fl * F;
                    lds_load_frag<F>(xs + row[rr], x[rr]);
                    lds_load_frag<F>(as + row[rr], a[rr]);
                }
                const int live = !LENGTHS ? NC : valid ? fused_live_rows<NC>(A, it, qg, len) : 0;
                if constexpr (HEADWISE) {
                    if (INVERSE) headwise_inverse_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x, a, wi, wj, A.tab, lane, slots, live);
                    else headwise_forward_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x, a, wi, wj, A.tab, lane, slots, live);
                } else {
                    if (INVERSE) inverse_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x, a, wi, wj, A.tab, lane, slots, live);
                    else forward_core<NC, EC, R, F, TANH_ONLY, LENGTHS, true>(x, a, wi, wj, A.tab, lane, slots, live);
                }
                if (valid) {
#pragma unroll
                    for (int rr = 0; rr < R; ++rr) {
                        if (LENGTHS && rl * R + rr >= live) continue;
                        lds_store_frag<F>(xs + row[rr], x[rr]);
                        lds_store_frag<F>(as + row[rr], a[rr]);
                    }
                }
            }
            __syncthreads();
        }
        // out of the scaled form
        fused_store_rows_scaled<NC, EC, NW, RADIX>(A, it, xs, A.tab.inv_kappa, A.out0, A.out_dtype, A.aux0);
        fused_store_rows_scaled<NC, EC, NW, RADIX>(A, it, as, INVERSE ? A.tab.inv_b_scale : A.tab.inv_a_scale, A.out1,
                                                   A.out_dtype, A.aux1);
        __syncthreads();
    }
}

template <int NC, int EC, int R, int F, bool TANH_ONLY, bool RADIX = false, bool LENGTHS = false, bool HEADWISE = false>
__global__ void __launch_bounds__(64 * kFusedWavesBwd, TANH_ONLY ? (R * F <= 8 ? 4 : 2) : 1) fused_backward_kernel(const FusedArgs A) {
    static_assert(!(RADIX && LENGTHS), "context lengths go with the stride permutation");
    constexpr int NW = kFusedWavesBwd;
    using T = Tile<NC, EC, R, F>;
    extern __shared__ float4 fused_lds4[];
    float* lds = reinterpret_cast<float*>(fused_lds4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fl = lane % T::LF, rl = (lane / T::LF) % T::LR, gw = lane / T::LPG;
    const uint32_t rows = A.window * NC;
    const float om = 1.0f - A.tab.m;
    float* ys = lds;
    float* bs = ys + rows * EC;
    float* gs = bs + rows * EC;
    float* ps = gs + rows * EC;                                  // p = (1-m) g + h
    float* w_lds = ps + rows * EC;                               // [kFusedMaxStages][2][EC]
    float* after = w_lds + kFusedMaxStages * 2 * EC;
    float4* slots = reinterpret_cast<float4*>(after) + wave * (F / 4) * 64;
    float* dw_all = after + (T::LR == 1 ? 0 : NW * F * 64);   // [wave][stage][2][EC]
    const int dw_wave_stride = A.n_stages * 2 * EC;
    float* dw_mine = dw_all + wave * dw_wave_stride;
    for (int k = lane; k < dw_wave_stride; k += 64) dw_mine[k] = 0.f;
    const int head = blockIdx.x % A.n_head;   // == head of every item of this workgroup (gridDim.x % n_head == 0)
    fused_load_weights<EC, NW>(A, head, w_lds);

    // The step code leaves no registers to carry a window across the stages, but between two items they are free:
    // the window of the next item is requested (all loads of a thread back to back) before the owned rows of this one
    // are written out, and lands in LDS after them.
    constexpr int K = (int)((kFusedStateBytesBwd / 4 / sizeof(float4) + 64 * NW - 1) / (64 * NW));
    struct Raw {
        uint4 y[K], b[K], g[K], h[K];
    };
    auto fetch = [&](uint32_t item, Raw& r) {
        int64_t off[K];
        fused_window_offsets<NC, EC, NW, K, RADIX>(A, fused_item<NC, EC, RADIX>(A, item), rows, off);
        fused_fetch_rows<K>(A.in0, A.in_dtype, off, r.y);
        fused_fetch_rows<K>(A.in1, A.in_dtype, off, r.b);
        fused_fetch_rows<K>(A.g0, A.g_dtype, off, r.g);
        fused_fetch_rows<K>(A.g1, A.g_dtype, off, r.h);
    };
    auto commit = [&](const Raw& r) {
        fused_commit_rows<NC, EC, NW, K>(r.y, A.in_dtype, ys, rows, A.tab.kappa);
        fused_commit_rows<NC, EC, NW, K>(r.b, A.in_dtype, bs, rows, A.tab.b_scale);
        fused_commit_rows<NC, EC, NW, K>(r.g, A.g_dtype, gs, rows, 1.0f);
        constexpr uint32_t CPR = EC / 4;   // p = (1-m) g + h  (h = 0 when dya is null: the fetch left zeros)
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t c = threadIdx.x + k * 64 * NW;
            if (c < rows * CPR) {
                float g[4], h[4];
                fused_raw_to_float(r.g[k], A.g_dtype, g);
                fused_raw_to_float(r.h[k], A.g_dtype, h);
#pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = fmaf(om, g[e], h[e]);
                lds_store_frag<4>(ps + fused_lds_place<NC>(c / CPR) * EC + (c % CPR) * 4, h);
            }
        }
    };
    if (blockIdx.x < A.total_items) {
        Raw first;
        fetch(blockIdx.x, first);
        commit(first);
    }
    __syncthreads();
    for (uint32_t item = blockIdx.x; item < A.total_items; item += gridDim.x) {
        const FusedItem it = fused_item<NC, EC, RADIX>(A, item);
        const int32_t len = LENGTHS ? max(0, min(A.ctx_len[it.batch], (int32_t)A.N)) : 0;
        for (int st = A.n_stages - 1; st >= 0; --st) {
            const uint32_t ss = A.sub_stride[st];
            const uint32_t ngroups = A.closed ? A.window : A.window - (NC - 1) * ss;
            float wi[F], wj[F], dwi[F], dwj[F];
            lds_load_frag<F>(w_lds + st * 2 * EC + fl * F, wi);
            lds_load_frag<F>(w_lds + st * 2 * EC + EC + fl * F, wj);
#pragma unroll
            for (int f = 0; f < F; ++f) dwi[f] = dwj[f] = 0.f;
            for (uint32_t wt = wave; wt * T::GPW < ngroups; wt += NW) {
                const uint32_t qg = wt * T::GPW + gw;
                const bool valid = qg < ngroups;
                const float own = (valid && qg - it.own_lo < it.own_cnt) ? 1.0f : 0.0f;  // unsigned: lo <= qg < lo+cnt
                float Y[R][F], B[R][F], G[R][F], P[R][F];
                uint32_t row[R];
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    row[rr] = fused_lds_row<NC, RADIX>(A, valid ? qg : 0u, rl * R + rr, ss) * EC + fl * F;
                    lds_load_frag<F>(ys + row[rr], Y[rr]);
                    lds_load_frag<F>(bs + row[rr], B[rr]);
                    lds_load_frag<F>(gs + row[rr], G[rr]);
                    lds_load_frag<F>(ps + row[rr], P[rr]);
                }
                const int live = !LENGTHS ? NC : valid ? fused_live_rows<NC>(A, it, qg, len) : 0;
                if (LENGTHS && live != NC) {
                    // G, P carry m^-t: the steps this group skips still count.  Rows past the length only take the
                    // factor of the whole stage and leave the sums of the group (zeros in the registers); the live
                    // rows take the factor of the skipped steps here and that of their own steps in the step code.
                    const float isc = pow_steps(A.tab.im, NC - live);
#pragma unroll
                    for (int rr = 0; rr < R; ++rr) {
                        const bool dead = rl * R + rr >= live;
#pragma unroll
                        for (int f = 0; f < F; ++f) {
                            const float sc = dead ? A.tab.inv_m_pow_n : isc;
                            G[rr][f] *= sc;
                            P[rr][f] *= sc;
                        }
                        if (dead) {
                            if (valid) {
                                lds_store_frag<F>(gs + row[rr], G[rr]);
                                lds_store_frag<F>(ps + row[rr], P[rr]);
                            }
#pragma unroll
                            for (int f = 0; f < F; ++f) Y[rr][f] = B[rr][f] = G[rr][f] = P[rr][f] = 0.f;
                        }
                    }
                }
                if constexpr (HEADWISE)
                    headwise_backward_core<NC, EC, R, F, true, TANH_ONLY, LENGTHS, true>(
                        Y, B, G, P, wi, wj, dwi, dwj, own, A.tab, (A.n_stages - 1 - st) * NC, lane, slots, live);
                else
                    backward_core<NC, EC, R, F, true, TANH_ONLY, LENGTHS, true>(Y, B, G, P, wi, wj, dwi, dwj, own, A.tab,
                                                                              (A.n_stages - 1 - st) * NC, lane, slots, live);
                if (valid) {
#pragma unroll
                    for (int rr = 0; rr < R; ++rr) {
                        if (LENGTHS && rl * R + rr >= live) continue;
                        lds_store_frag<F>(ys + row[rr], Y[rr]);
                        lds_store_frag<F>(bs + row[rr], B[rr]);
                        lds_store_frag<F>(gs + row[rr], G[rr]);
                        lds_store_frag<F>(ps + row[rr], P[rr]);
                    }
                }
            }
            // this wave's dW share of the stage: sum the lanes of each half of the wave that hold the same features,
            // then the two halves add to the wave's slot one after the other (a wave's LDS operations keep their
            // order: the sum is the same in every run, and the costly exchange across the halves is not needed)
#pragma unroll
            for (int f = 0; f < F; ++f) {
                dwi[f] = lane_sum<T::LF, 32, true>(dwi[f]);
                dwj[f] = lane_sum<T::LF, 32, true>(dwj[f]);
            }
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                if (lane == fl + 32 * half) {
                    float* d = dw_mine + st * (2 * EC) + fl * F;
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        d[f] += dwi[f];
                        d[EC + f] += dwj[f];
                    }
                }
            }
            __syncthreads();
        }
        auto write_out = [&]() {   // owned rows back to true values: g = G m^T, h = P m^T - (1-m) g, x = xs / kappa, xa = bh / b_scale
            constexpr uint32_t CPR = EC / 4;
            const uint32_t r0 = it.own_lo * NC, nrows = it.own_cnt * NC;
            for (uint32_t c = threadIdx.x; c < nrows * CPR; c += 64 * NW) {
                const uint32_t lr = r0 + c / CPR, c4 = c % CPR;
                const int64_t off = fused_row_offset<NC, RADIX>(A, it, lr) + c4 * 4;
                float g[4], h[4];
                lds_load_frag<4>(gs + fused_lds_place<NC>(lr) * EC + c4 * 4, g);
                lds_load_frag<4>(ps + fused_lds_place<NC>(lr) * EC + c4 * 4, h);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    g[k] *= A.scale_dn;
                    h[k] = fmaf(h[k], A.scale_dn, -om * g[k]);
                }
                store_frag<4>(A.out0, A.out_dtype, off, true, g);
                store_frag<4>(A.out1, A.out_dtype, off, true, h);
            }
            if (A.aux0) {
                fused_store_rows_scaled<NC, EC, NW, RADIX>(A, it, ys, A.tab.inv_kappa, A.aux0, NCN_F32, nullptr);
                fused_store_rows_scaled<NC, EC, NW, RADIX>(A, it, bs, A.tab.inv_b_scale, A.aux1, NCN_F32, nullptr);
            }
        };
        if (item + gridDim.x < A.total_items) {   // the same for the whole workgroup
            Raw next;
            fetch(item + gridDim.x, next);
            write_out();
            __syncthreads();   // every thread has read what it writes out: the window may be overwritten
            commit(next);
        } else {
            write_out();
        }
        __syncthreads();
    }
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
