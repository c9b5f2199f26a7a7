// The reversible backward kernels for heads of one feature (see ncn_headwise.hip).
#define NCN_HEADWISE_BACKWARD 1
#include "ncn_headwise.hip"
