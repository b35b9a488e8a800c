// The gate/up launch whose two projections have different formats (block-FP8 and NVFP4): both GEMV cores in one
// translation unit.
#define DGPP_GEMV_IMPL
#define DGPP_GEMV_MIXED
#include "gemv_kernels.hpp"
