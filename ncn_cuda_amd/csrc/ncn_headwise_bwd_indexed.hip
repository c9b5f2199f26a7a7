// The table / radix / context-length build of the backward kernels for heads of one feature (see ncn_headwise.hip).
#define NCN_INDEXED_BUILD 1
#define NCN_HEADWISE_BACKWARD 1
#include "ncn_headwise.hip"
