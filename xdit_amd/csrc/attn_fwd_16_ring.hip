// The 16-bit attention forward as a ring step (see attn_fwd_16_impl.h): the kernels whose epilogue
// folds the block into the fp32 accumulator of the ring, built apart from the others so that
// neither epilogue costs the other registers.
#include "attn_fwd_16_impl.h"

namespace xdit {

// Host-side launcher (called from the C ABI after argument validation; p.acc_out != nullptr).
hipError_t launch_attn_fwd_16_ring(const AttnParams& p, int dtype_is_fp16, int D, int rows_per_block, hipStream_t stream) {
  return dtype_is_fp16 ? launch_typed<_Float16, true>(p, D, rows_per_block, stream) : launch_typed<__bf16, true>(p, D, rows_per_block, stream);
}

}  // namespace xdit
