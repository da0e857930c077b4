// Shared device-side types and helpers for the gfx950 attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "attn_walk.h"

namespace xdit {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;

#define XDIT_LDS __attribute__((address_space(3)))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Parameters of one attention-forward launch (passed by value).
struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  const void* k2;
  const void* v2;
  void* out;
  float* lse;
  int64_t qs_b, qs_h, qs_s;
  int64_t ks_b, ks_h, ks_s;
  int64_t vs_b, vs_h, vs_s;
  int64_t k2s_b, k2s_h, k2s_s;
  int64_t v2s_b, v2s_h, v2s_s;
  int64_t os_b, os_h, os_s;
  int64_t ls_b, ls_h;
  const float* q_descale;
  const float* k_descale;
  const float* v_descale;
  int64_t ds_b, ds_h;
  int B, H;
  int Sq, Sk, Sk2;
  int nq_tiles;       // ceil(Sq / rows per workgroup)
  int total_tiles;    // B * H * nq_tiles
  int tiles_per_xcd;  // ceil(total_tiles / 8)
  float scale;        // softmax scale
  int d_actual;       // head_dim of the tensors when the kernel is built for a larger one (0: the kernel's own)
  int cu_count;       // compute units the launch is planned for (0: those of the current device)
  // balanced launch (see attn_fwd_16_kernel); all zero for a plain launch
  int split_full;     // query tiles handled whole, by the first workgroups
  int split_units;    // workgroups sharing the KV iterations of the remaining query tiles
  int split_len;      // KV iterations per such workgroup
  int split_pmax;     // workspace slots per remaining query tile
  int split_fuse0;    // first workgroup that takes a range after its own query tile (> split_full: none)
  int split_share;    // KV iterations of the remaining query tiles per resident workgroup
  int split_claimers; // workgroups that process ranges
  unsigned* split_counter;  // ranges handed out beyond the first of every claimer (nullptr: one range each);
                            // streamed sharing: one counter of KV iterations per shared tile
  int split_dyn;      // streamed sharing of the remaining tiles (see WorkgroupWalk)
  int split_s0;       // KV iterations every member of a tile's group owns before it draws from the counter
  int streamed_ok;    // the caller opted in to streamed sharing (results then reproducible to rounding only)
  int split_order;    // claimers process their range BEFORE their whole query tile (see WorkgroupWalk)
  int split_fold;     // the parts of a shared tile are folded inside the attention kernel (fold duties, attn_walk.h)
  int split_policy;   // 1: plain launch; 2: balance whenever the plan shortens the critical path by kMinSaving iterations
  // ring step (optional): the result is folded into an fp32 accumulator in the epilogue
  float* acc_out;     // (B,H,Sq,D) fp32 running output, nullptr: plain forward
  float* acc_lse;     // (B,H,Sq) fp32 running log-sum-exp
  int64_t ao_b, ao_h, ao_s;
  int64_t al_b, al_h, al_s;
  int acc_first;      // initialise the accumulator from this block instead of folding
  int acc_store;      // write acc_out back (0: only `out` and acc_lse receive the result)
  unsigned* ws_counters;  // workspace: its counter region (start of the workspace)
  int ws_preserved;   // the caller vouches that the counter region is as this library's last call left it
  void* ws_out;       // workspace: partial outputs [tile][slot][row][D] in the output dtype ...
  float* ws_lse;      // ... followed by partial log-sum-exps [tile][slot][row]
  size_t ws_bytes;
};

// Combine a value across the two 32-lane halves of a wavefront (lane l with lane l^32).
// v_permlane32_swap(a, b) leaves {own a, other half's a} in the low half and
// {other half's b, own b} in the high half, so with a == b both halves hold {own, other}.
__device__ __forceinline__ float max_halves(float x) {
  int xi = __builtin_bit_cast(int, x);
  auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  return fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
}
__device__ __forceinline__ float sum_halves(float x) {
  int xi = __builtin_bit_cast(int, x);
  auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

// The two functions of the ring fold, shared by the merge kernel and the fused epilogue so that
// both give the same bits.  logsigmoid(x) = min(x, 0) - log1p(exp(-|x|)), the form torch evaluates.
__device__ __forceinline__ float log_sigmoid(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}
__device__ __forceinline__ float sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
// acc - w * (acc - blk), with the rounding of one fused multiply-add.
__device__ __forceinline__ float fold_value(float acc, float blk, float w) {
  return __builtin_fmaf(-w, acc - blk, acc);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

}  // namespace xdit
