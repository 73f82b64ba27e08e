// The block-wise kernels of uvu_big.hip instantiated with one factor per weight path; see uvu_kernels_ps.hip.
#define CGTP_UVU_PS_UNIT
#include "uvu_big.hip"
