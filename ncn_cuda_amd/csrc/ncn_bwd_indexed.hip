// The backward stage kernels built to read a grouping table and context lengths (see ncn_bwd.hip).
#define NCN_INDEXED_BUILD 1
#include "ncn_bwd.hip"
