// The table / context-length build of the backward stage kernels without a loop over tiles (see ncn_bwd.hip).
#define NCN_INDEXED_BUILD 1
#define NCN_ONCE_BUILD 1
#include "ncn_bwd.hip"
