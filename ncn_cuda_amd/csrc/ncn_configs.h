// The shapes the register kernels are built for: X(n_cache, head width, R, F) where each lane holds an
// R-row x F-feature register tile of its group (see ncn_stage_kernels.h).  One entry per (n_cache, head width).
// 16 elements per lane (R = 4, F = 4) keeps the backward kernel at 128 VGPRs (4 waves per SIMD); larger
// tiles are only used where a group would otherwise not fit the 64 lanes of a wavefront.
#pragma once
#define NCN_FOR_EACH_FAST_CONFIG(X) \
    X(2, 4, 2, 4) X(4, 4, 2, 4) X(8, 4, 4, 4) X(16, 4, 4, 4) X(32, 4, 4, 4) X(64, 4, 4, 4) \
    X(2, 8, 2, 4) X(4, 8, 2, 4) X(8, 8, 4, 4) X(16, 8, 4, 4) X(32, 8, 4, 4) X(64, 8, 4, 4) \
    X(2, 16, 2, 4) X(4, 16, 2, 4) X(8, 16, 4, 4) X(16, 16, 4, 4) X(32, 16, 4, 4) X(64, 16, 4, 4) \
    X(2, 32, 2, 4) X(4, 32, 2, 4) X(8, 32, 4, 4) X(16, 32, 4, 4) X(32, 32, 4, 4) X(64, 32, 4, 8) \
    X(2, 64, 2, 8) X(4, 64, 2, 8) X(8, 64, 4, 8) X(16, 64, 4, 8) X(32, 64, 4, 8) \
    X(2, 128, 2, 8) X(4, 128, 2, 8) X(8, 128, 4, 8) X(16, 128, 4, 8)

// The shapes X(n_cache, head width) with multi-stage (LDS-resident) builds, under the stride permutation, with context
// lengths and for the radix-n levels alike.  Groups of 8 rows and more are bound by arithmetic even stage by stage
// (measured 10 % slower through LDS) and have none.
#define NCN_FOR_EACH_FUSED_CONFIG(X) \
    X(2, 8) X(4, 8) X(2, 16) X(4, 16) X(2, 32) X(4, 32) X(2, 64) X(4, 64) X(2, 128) X(4, 128)
