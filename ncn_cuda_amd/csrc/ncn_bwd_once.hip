// The backward stage kernels in their form without a loop over tiles (see ncn_bwd.hip).
#define NCN_ONCE_BUILD 1
#include "ncn_bwd.hip"
