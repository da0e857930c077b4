// Host-side launch functions of the kernels, shared between the kernel files and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"

namespace xdit {

// Parameters of one merge launch (passed by value to the kernel).
struct MergeParams {
  float* acc_out;
  float* acc_lse;
  const void* block_out;
  const float* block_lse;
  void* final_out;
  int64_t ao_b, ao_h, ao_s;
  int64_t bo_b, bo_h, bo_s;
  int64_t fo_b, fo_h, fo_s;
  int64_t al_b, al_h, al_s;
  int64_t bl_b, bl_h, bl_s;
  int B, H, S, D;
  int first;
  int64_t rows;  // B * H * S
};

// Parameters of one fp8 quantiser call.  `amax` and `descale` are the same (B,H) fp32 buffer:
// it holds the abs-max values between the passes and the descales at the end.
struct QuantParams {
  const void* x;
  void* y;
  float* amax;
  float* descale;
  const float* scale_in;  // optional static scale (one float); skips the abs-max pass
  int64_t xs_b, xs_h, xs_s;
  int64_t ys_b, ys_h, ys_s;
  int B, H, S, D;
  int per_tensor;
  int had_block;    // Hadamard rotation block along head_dim (<= 1: none)
  float had_scale;  // 1/sqrt(had_block) in fp32; the kernel rounds it to the input dtype
  // optional second tensor (B,H,S2,D) quantised with the scales of the first
  const void* x2;
  void* y2;
  int64_t x2s_b, x2s_h, x2s_s;
  int64_t y2s_b, y2s_h, y2s_s;
  int S2;
  // optional scratch: partial_slots floats, one per workgroup of the abs-max pass
  float* partials;
  int64_t partial_slots;
};

// Parameters of one prologue launch (RMSNorm + rotary embedding + re-layout of Q or K).
struct PrologueParams {
  const void* x;
  void* y;
  const void* weight;  // gain in the tensor's dtype: D entries (norm 1) or H*D (norm 2); may be null
  const float* cos;
  const float* sin;
  int64_t xs_b, xs_h, xs_s;
  int64_t ys_b, ys_h, ys_s;
  int64_t rope_stride;  // elements between rows of cos / sin
  int64_t rows;         // B * S * H
  int B, H, S, D;
  int norm;             // 0 none, 1 over head_dim per head, 2 over all heads of a token
  int rope_mode;        // 0 none, 1 interleaved pairs, 2 split halves, 3 interleaved pairs, Wan's table indexing
  int rope_row0, rope_rows;  // rows [row0, row0 + rows) of S are rotated, with table row s - row0
  int lpr;              // lanes per row: smallest power of two >= D/8
  float eps, inv_n;     // inv_n = 1 / number of elements under one norm statistic
};

// Up to kPrologueBatchMax prologue jobs of one dtype for a single launch.
constexpr int kPrologueBatchMax = 8;
struct PrologueBatch {
  PrologueParams job[kPrologueBatchMax];
  int n;
};

// dtype codes below are the C ABI's xdit_dtype values: 0 bf16, 1 fp16, 2 fp32, 3 fp8 e4m3fn.
hipError_t launch_attn_fwd_16(const AttnParams& p, int dtype_is_fp16, int D, int rows_per_block, hipStream_t stream);
hipError_t launch_attn_fwd_16_ring(const AttnParams& p, int dtype_is_fp16, int D, int rows_per_block, hipStream_t stream);  // p.acc_out set
size_t attn_fwd_16_workspace(const AttnParams& p, int D, int rows_per_block, AttnParams* plan = nullptr, bool fold_only = false);  // fold_only: the ring step
hipError_t launch_attn_fwd_fp8(const AttnParams& p, int D, int out_is_fp16, int rows_per_block, hipStream_t stream);  // D: 128 or 64
size_t attn_fwd_fp8_workspace(const AttnParams& p, int D, int rows_per_block, AttnParams* plan = nullptr, bool fold_only = false);
hipError_t launch_attn_fwd_f32(const AttnParams& p, int D, hipStream_t stream);  // fp32 tensors only
int attn_fwd_f32_rows(const AttnParams& p);  // query rows per workgroup the fp32 launch takes: 128, or 64 (64-key tiles split between wavefront pairs)
hipError_t launch_fp8_quant(const QuantParams& p, int in_dtype, hipStream_t stream);
hipError_t launch_qk_prologue(const PrologueParams& p, int dtype, hipStream_t stream);
hipError_t launch_qk_prologue_batch(const PrologueBatch& b, int dtype, hipStream_t stream);
int prologue_max_token_elems();
hipError_t launch_lse_merge(const MergeParams& p, int block_dtype, int final_dtype, hipStream_t stream);

}  // namespace xdit
