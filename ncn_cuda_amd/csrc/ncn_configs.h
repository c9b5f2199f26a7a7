// The (n_cache, head width, features per lane) triples the register kernels are built for.
// Must agree with fast_fpl() in ncn_launch.h (checked by static_asserts where the list is expanded).
#pragma once
#define NCN_FOR_EACH_FAST_CONFIG(X)                                   \
    X(2, 4, 4) X(4, 4, 4) X(8, 4, 4) X(16, 4, 4) X(32, 4, 4)          \
    X(2, 8, 8) X(4, 8, 8) X(8, 8, 8) X(16, 8, 8) X(32, 8, 8)          \
    X(2, 16, 16) X(4, 16, 16) X(8, 16, 16) X(16, 16, 16) X(32, 16, 16) \
    X(2, 32, 16) X(4, 32, 16) X(8, 32, 16) X(16, 32, 16) X(32, 32, 16) \
    X(2, 64, 16) X(4, 64, 16) X(8, 64, 16) X(16, 64, 16)
