// The table-driven matrix-core kernels of the fully connected products (uvt_kernels.hip) in double precision; a
// translation unit of its own so that the two sets compile side by side.
#define CGTP_UVT_F64
#include "uvt_kernels.hip"
