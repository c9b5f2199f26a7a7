// The forward and inverse stage kernels built to read a grouping table and context lengths (see ncn_fwd.hip).
#define NCN_INDEXED_BUILD 1
#include "ncn_fwd.hip"
