// The 16-bit attention forward (see attn_fwd_16_impl.h): the kernels that write the output (or the
// partial results of a balanced launch), their launcher and the workspace planning.
#include "attn_fwd_16_impl.h"

namespace xdit {

// Workspace bytes a balanced launch of this problem would use (0: none needed); `plan`, if given,
// receives the launch geometry (as if that workspace were supplied).
template <int D, int NW>
static size_t workspace_one(const AttnParams& p, AttnParams* plan, bool fold_only) {
  AttnParams q = p;
  constexpr int rows = 32 * NW;
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  const size_t need = plan_split(q, rows, resident_workgroups(NW, p.cu_count), D, 2, kClaimsPerWorkgroup, true, fold_only);
  if (plan != nullptr) *plan = q;
  return need;
}

size_t attn_fwd_16_workspace(const AttnParams& p, int D, int rows_per_block, AttnParams* plan, bool fold_only) {
  if (D == 128 && rows_per_block == 384) return workspace_one<128, 12>(p, plan, fold_only);
  if (D == 128 && rows_per_block == 256) return workspace_one<128, 8>(p, plan, fold_only);
  if (D == 128) return workspace_one<128, 4>(p, plan, fold_only);
  if (D == 64 && rows_per_block == 384) return workspace_one<64, 12>(p, plan, fold_only);
  if (D == 64 && rows_per_block == 256) return workspace_one<64, 8>(p, plan, fold_only);
  if (D == 64) return workspace_one<64, 4>(p, plan, fold_only);
  return 0;
}

// Host-side launcher (called from the C ABI after argument validation; p.acc_out == nullptr).
hipError_t launch_attn_fwd_16(const AttnParams& p, int dtype_is_fp16, int D, int rows_per_block, hipStream_t stream) {
  return dtype_is_fp16 ? launch_typed<_Float16, false>(p, D, rows_per_block, stream) : launch_typed<__bf16, false>(p, D, rows_per_block, stream);
}

}  // namespace xdit
