// The context-length build of the multi-stage passes for heads of one feature (see ncn_fused_headwise.hip).
#define NCN_LENGTHS_BUILD 1
#include "ncn_fused_headwise.hip"
