// Instantiates the GEMV-core kernels for one weight format (kFmtFp8F32).
#define DGPP_GEMV_IMPL
#define DGPP_GEMV_PAIR
#include "gemv_kernels.hpp"
#include "gemv_chain.hpp"

namespace dgpp_amd {
template hipError_t launch_dense_fmt<kFmtFp8F32>(const DenseArgs&, hipStream_t);
template hipError_t launch_dense_multi_fmt<kFmtFp8F32>(const DenseArgs*, int, hipStream_t);
template hipError_t launch_slot_gate_up_fmt<kFmtFp8F32>(const SlotArgs&, hipStream_t);
template hipError_t launch_select_gate_up_fmt<kFmtFp8F32>(const SlotArgs&, const SelectArgs&, hipStream_t);
template hipError_t launch_slot_down_fmt<kFmtFp8F32>(const SlotArgs&, hipStream_t);
template hipError_t launch_grouped_fmt<kFmtFp8F32>(const GroupedArgs&, int, int, hipStream_t);
template hipError_t launch_dense_mma_fmt<kFmtFp8F32>(const DenseArgs&, float*, size_t, hipStream_t);
template hipError_t launch_grouped_mma_fmt<kFmtFp8F32>(const GroupedArgs&, int, int, hipStream_t);
template hipError_t launch_token_down_fmt<kFmtFp8F32>(const TokenDownArgs&, hipStream_t);
template hipError_t launch_slot_chain_fmt<kFmtFp8F32>(const ChainArgs&, const SelectArgs*, hipStream_t);
}  // namespace dgpp_amd
