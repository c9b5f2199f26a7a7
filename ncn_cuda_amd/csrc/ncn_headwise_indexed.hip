// The table / radix / context-length build of the forward and inverse kernels for heads of one feature (see
// ncn_headwise.hip).
#define NCN_INDEXED_BUILD 1
#include "ncn_headwise.hip"
