// Instantiates the GEMV-core kernels for one weight format (kFmtNvfp4).
#define DGPP_GEMV_IMPL
#include "gemv_kernels.hpp"
#include "gemv_chain.hpp"

namespace dgpp_amd {
template hipError_t launch_dense_fmt<kFmtNvfp4>(const DenseArgs&, hipStream_t);
template hipError_t launch_slot_gate_up_fmt<kFmtNvfp4>(const SlotArgs&, hipStream_t);
template hipError_t launch_select_gate_up_fmt<kFmtNvfp4>(const SlotArgs&, const SelectArgs&, hipStream_t);
template hipError_t launch_slot_down_fmt<kFmtNvfp4>(const SlotArgs&, hipStream_t);
template hipError_t launch_grouped_fmt<kFmtNvfp4>(const GroupedArgs&, int, int, hipStream_t);
template hipError_t launch_dense_mma_fmt<kFmtNvfp4>(const DenseArgs&, float*, size_t, hipStream_t);
template hipError_t launch_grouped_mma_fmt<kFmtNvfp4>(const GroupedArgs&, int, int, hipStream_t);
template hipError_t launch_token_down_fmt<kFmtNvfp4>(const TokenDownArgs&, hipStream_t);
template hipError_t launch_slot_chain_fmt<kFmtNvfp4>(const ChainArgs&, const SelectArgs*, hipStream_t);
}  // namespace dgpp_amd
