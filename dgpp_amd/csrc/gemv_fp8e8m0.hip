// Instantiates the dense GEMV for FP8 payloads with an E8M0 byte scale grid (MXFP8). The
// expert-view table has no E8M0 field, so there are no slot / grouped forms of this format.
#define DGPP_GEMV_IMPL
#include "gemv_kernels.hpp"

namespace dgpp_amd {
template hipError_t launch_dense_fmt<kFmtFp8E8M0>(const DenseArgs&, hipStream_t);
template hipError_t launch_dense_multi_fmt<kFmtFp8E8M0>(const DenseArgs*, int, hipStream_t);
template hipError_t launch_dense_mma_fmt<kFmtFp8E8M0>(const DenseArgs&, float*, size_t, hipStream_t);
}  // namespace dgpp_amd
