// The channel-wise tensor-product kernels of uvu_kernels.hip instantiated with one factor per weight path (a table
// that differs from the compiled one by its path / channel normalisation); a translation unit of its own so that the
// two sets of kernels compile in parallel.
#define CGTP_UVU_PS_UNIT
#include "uvu_kernels.hip"
