// Fused ring online-softmax merge (one pass over HBM, fp32 arithmetic) for gfx950.
//
//   acc_out <- acc_out - sigmoid(block_lse - acc_lse) * (acc_out - block_out)
//   acc_lse <- acc_lse - logsigmoid(acc_lse - block_lse)
//
// This is the formula torch's _SDPAMerger._merge_one uses
// (torch/distributed/tensor/experimental/_context_parallel/_attention.py:181-182) and that
// xDiT's legacy ring loop reaches through `update_out_and_lse`
// (xfuser/core/long_ctx_attention/ring/ring_flash_attn.py:138).  `first` initialises the
// accumulator from the block instead (the `out is None` branch of update_out_and_lse /
// _attention.py:161-163), and `final_out`, when given, receives the merged rows in the block
// dtype (the epilogue cast at ring_flash_attn.py:145) in the same pass.
//
// Memory-bound: a thread moves 8 consecutive head_dim elements (32 B of fp32 accumulator, 16 B
// of 16-bit block) at a time; the D/8 chunks of a row are held by adjacent lanes of ONE
// wavefront (MergeMap in attn_walk.h), so accumulator accesses coalesce to full rows and a
// wavefront covers whole rows only.  Every lane of a row reads the row's accumulated
// log-sum-exp before the row's first lane overwrites it in place; with the row inside one
// wavefront, program order guarantees that for every head_dim (rows that straddled two
// wavefronts, as they would at head_dim 72 with a flat thread -> chunk map, could see the new
// value in the later wavefront).
#include "common.h"
#include "launchers.h"

namespace xdit {

template <typename T> struct Load8;
template <> struct Load8<float> {
  static __device__ __forceinline__ void ld(const void* p, float (&x)[8]) {
    const f32x4* q = (const f32x4*)p;
    f32x4 a = q[0], b = q[1];
    for (int i = 0; i < 4; i++) { x[i] = a[i]; x[4 + i] = b[i]; }
  }
  static __device__ __forceinline__ void st(void* p, const float (&x)[8]) {
    f32x4 a = {x[0], x[1], x[2], x[3]}, b = {x[4], x[5], x[6], x[7]};
    ((f32x4*)p)[0] = a;
    ((f32x4*)p)[1] = b;
  }
};
template <> struct Load8<__bf16> {
  static __device__ __forceinline__ void ld(const void* p, float (&x)[8]) {
    bf16x8 v = *(const bf16x8*)p;
    for (int i = 0; i < 8; i++) x[i] = (float)v[i];
  }
  static __device__ __forceinline__ void st(void* p, const float (&x)[8]) {
    bf16x8 v;
    for (int i = 0; i < 8; i++) v[i] = (__bf16)x[i];
    *(bf16x8*)p = v;
  }
};
template <> struct Load8<_Float16> {
  static __device__ __forceinline__ void ld(const void* p, float (&x)[8]) {
    f16x8 v = *(const f16x8*)p;
    for (int i = 0; i < 8; i++) x[i] = (float)v[i];
  }
  static __device__ __forceinline__ void st(void* p, const float (&x)[8]) {
    f16x8 v;
    for (int i = 0; i < 8; i++) v[i] = (_Float16)x[i];
    *(f16x8*)p = v;
  }
};

template <typename TB, typename TF, bool HAS_FINAL>
__global__ __launch_bounds__(256) void lse_merge_kernel(const MergeParams p, const MergeMap map) {
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  int64_t row;
  int chunk0;
  if (!merge_thread_row(map, wave, threadIdx.x & 63, row, chunk0) || row >= p.rows) return;
  // row -> (b, h, s); consecutive rows walk s fastest, then h, then b
  const int s = (int)(row % p.S);
  const int64_t bh = row / p.S;
  const int h = (int)(bh % p.H);
  const int b = (int)(bh / p.H);

  const float* bl = p.block_lse + b * p.bl_b + h * p.bl_h + s * p.bl_s;
  float* al = p.acc_lse + b * p.al_b + h * p.al_h + s * p.al_s;
  float* ao_row = p.acc_out + b * p.ao_b + h * p.ao_h + s * p.ao_s;
  const TB* bo_row = (const TB*)p.block_out + b * p.bo_b + h * p.bo_h + s * p.bo_s;

  const int col = chunk0 * 8;  // head_dim <= 512: a lane holds one chunk
  float xb[8], xo[8];
  Load8<TB>::ld(bo_row + col, xb);
  const float blse = *bl;
  float new_lse;
  if (p.first) {
#pragma unroll
    for (int i = 0; i < 8; i++) xo[i] = xb[i];
    new_lse = blse;
  } else {
    Load8<float>::ld(ao_row + col, xo);
    const float lse = *al;  // read by every lane of the row before its first lane stores below
    const float w = sigmoid(blse - lse);
#pragma unroll
    for (int i = 0; i < 8; i++) xo[i] = fold_value(xo[i], xb[i], w);
    new_lse = lse - log_sigmoid(lse - blse);
  }
  Load8<float>::st(ao_row + col, xo);
  if (HAS_FINAL) {
    TF* fo = (TF*)p.final_out + b * p.fo_b + h * p.fo_h + s * p.fo_s + col;
    Load8<TF>::st(fo, xo);
  }
  if (chunk0 == 0) *al = new_lse;
}

template <typename TB>
static hipError_t launch_tb(const MergeParams& p, int final_dtype, hipStream_t stream) {
  const MergeMap map = merge_map(p.D);
  const int64_t waves = (p.rows + map.rows_per_wave - 1) / map.rows_per_wave;
  if ((waves + 3) / 4 > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  if (p.final_out == nullptr) {
    hipLaunchKernelGGL((lse_merge_kernel<TB, float, false>), grid, block, 0, stream, p, map);
  } else if (final_dtype == 0) {
    hipLaunchKernelGGL((lse_merge_kernel<TB, __bf16, true>), grid, block, 0, stream, p, map);
  } else if (final_dtype == 1) {
    hipLaunchKernelGGL((lse_merge_kernel<TB, _Float16, true>), grid, block, 0, stream, p, map);
  } else {
    hipLaunchKernelGGL((lse_merge_kernel<TB, float, true>), grid, block, 0, stream, p, map);
  }
  return hipGetLastError();
}

// dtype codes: 0 bf16, 1 fp16, 2 fp32 (the C ABI's xdit_dtype values).
hipError_t launch_lse_merge(const MergeParams& p, int block_dtype, int final_dtype, hipStream_t stream) {
  if (block_dtype == 0) return launch_tb<__bf16>(p, final_dtype, stream);
  if (block_dtype == 1) return launch_tb<_Float16>(p, final_dtype, stream);
  if (block_dtype == 2) return launch_tb<float>(p, final_dtype, stream);
  return hipErrorInvalidValue;
}

}  // namespace xdit
