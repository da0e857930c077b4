// fp8 (OCP e4m3fn) quantiser with abs-max scaling for gfx950: the step in front of the fp8
// attention kernel.  Restates per_tensor_quant (xfuser/core/distributed/attention_backend.py:606-615):
//     scale = absmax(x) / 448 ;  y = fp8(x / scale) ;  descale = scale broadcast to (B, H)
// with the abs-max taken over the whole tensor (`per_tensor`) or per (batch, head) slice, or a
// caller-supplied static scale.  With a scratch buffer of the caller: two launches on the
// caller's stream, (1) abs-max reduction, every workgroup storing its maximum in a scratch slot
// of its own, (2) scale and cast, every workgroup folding its slice's partial maxima first and
// the first one of a slice storing the descale; a static scale needs launch (2) only.  Without
// scratch: four launches, (1) clear the (B,H) abs-max buffer (a fill kernel, so the sequence can
// be captured in a HIP graph), (2) abs-max reduction with one atomic max per workgroup, (3) scale
// and cast, (4) turn the abs-max buffer into the descale values.  An optional second tensor (the
// joint keys or values) shares the scales of the first.  Both tensor passes are HBM-bound and read
// 16 bytes per lane; the division is a true fp32 division so results match the reference's
// `x / scale` bit for bit.  Optionally both passes first rotate each row along head_dim by a
// block Hadamard matrix (_fp8_hadamard_rotate, attention_backend.py:703-714), in registers.
#include "common.h"
#include "launchers.h"

namespace xdit {

namespace quant {

constexpr float kFp8Max = 448.0f;

template <typename T> __device__ __forceinline__ void load8(const T* p, float (&x)[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&x)[8]) {
  f32x4 a = ((const f32x4*)p)[0], b = ((const f32x4*)p)[1];
  for (int i = 0; i < 4; i++) { x[i] = a[i]; x[4 + i] = b[i]; }
}
template <> __device__ __forceinline__ void load8<__bf16>(const __bf16* p, float (&x)[8]) {
  bf16x8 v = *(const bf16x8*)p;
  for (int i = 0; i < 8; i++) x[i] = (float)v[i];
}
template <> __device__ __forceinline__ void load8<_Float16>(const _Float16* p, float (&x)[8]) {
  f16x8 v = *(const f16x8*)p;
  for (int i = 0; i < 8; i++) x[i] = (float)v[i];
}

// Rotates the rows by the Sylvester-Hadamard matrix of size `block` along head_dim, in place in
// the 8-element chunks the threads hold: the three butterfly levels inside a chunk in
// registers, the levels across chunks by exchanging with the lane that holds chunk c ^ m of the
// same row (the chunks of a block sit in consecutive, block-aligned lanes of one wavefront).
// Entries are +-r with r = `scale` rounded to T and the result is rounded to T, like the output
// of a matmul with the matrix held in T.  `c` is the chunk's index within its row.
template <typename T>
__device__ __forceinline__ void hadamard_rows(float (&v)[8], int block, float scale, int c) {
  if (block >= 2) {
#pragma unroll
    for (int j = 0; j < 8; j += 2) { const float a = v[j], b = v[j + 1]; v[j] = a + b; v[j + 1] = a - b; }
  }
  if (block >= 4) {
#pragma unroll
    for (int j = 0; j < 8; j += 4) {
#pragma unroll
      for (int i = 0; i < 2; i++) { const float a = v[j + i], b = v[j + i + 2]; v[j + i] = a + b; v[j + i + 2] = a - b; }
    }
  }
  if (block >= 8) {
#pragma unroll
    for (int i = 0; i < 4; i++) { const float a = v[i], b = v[i + 4]; v[i] = a + b; v[i + 4] = a - b; }
  }
  for (int m = 1; m * 8 < block; m <<= 1) {
    const bool upper = (c & m) != 0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float o = __shfl_xor(v[j], m);
      v[j] = upper ? o - v[j] : v[j] + o;
    }
  }
  const float r = (float)(T)scale;
#pragma unroll
  for (int j = 0; j < 8; j++) v[j] = (float)(T)(v[j] * r);
}

__global__ void fill_zero_kernel(float* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// Both tensor passes: grid = (blocks per slice, B*H).  A row of D elements is held by D/8
// consecutive threads (8 elements each), a workgroup covers 256 / (D/8) rows per step and every
// thread keeps kRowsInFlight rows in flight; rows advance by whole grid steps, so there is no
// division in the loop and the trip count is the same for every thread of a workgroup (the
// lanes of a row exchange data in the Hadamard rotation).
constexpr int kRowsInFlight = 4;
constexpr int kAbsmaxRowsInFlight = 8;  // the read-only pass: nothing but loads to keep in flight

template <typename T, int kRowsInFlight = quant::kRowsInFlight, typename F>
__device__ __forceinline__ void for_each_chunk(const QuantParams& p, const T* x, int64_t S, int64_t xs_s, F&& f) {
  const int cpr = p.D >> 3;
  const int rpb = 256 / cpr;              // rows per workgroup step
  const int c = threadIdx.x % cpr;
  const int r = threadIdx.x / cpr;
  const bool lane_live = r < rpb;
  const int64_t step = (int64_t)gridDim.x * rpb;
  for (int64_t base = (int64_t)blockIdx.x * rpb; base < S; base += step * kRowsInFlight) {
    float v[kRowsInFlight][8];
    int64_t s[kRowsInFlight];
#pragma unroll
    for (int j = 0; j < kRowsInFlight; j++) {
      s[j] = base + j * step + r;
      const int64_t sc = s[j] < S ? s[j] : S - 1;  // rows past the end re-read the last row
      load8<T>(x + sc * xs_s + c * 8, v[j]);
    }
#pragma unroll
    for (int j = 0; j < kRowsInFlight; j++) {
      if (p.had_block > 1) hadamard_rows<T>(v[j], p.had_block, p.had_scale, c);
      f(v[j], s[j], c, lane_live && s[j] < S);
    }
  }
}

// Maximum of a value over the workgroup (256 threads), returned to every thread.
__device__ __forceinline__ float block_max(float m) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  __shared__ float wm[4];
  __syncthreads();  // a previous use of wm is over
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
  __syncthreads();
  return fmaxf(fmaxf(wm[0], wm[1]), fmaxf(wm[2], wm[3]));
}

// Abs-max of a (batch, head) slice over both tensors.  With `partials` every workgroup stores
// its maximum in a slot of its own (no clearing, no atomics); otherwise one atomic max per
// workgroup goes to the slice's entry of the (cleared) amax buffer.
template <typename T>
__global__ __launch_bounds__(256) void absmax_kernel(const QuantParams p) {
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh - b * p.H;
  float m = 0.f;
  auto take = [&](float (&v)[8], int64_t, int, bool live) {
    if (live) {
#pragma unroll
      for (int j = 0; j < 8; j++) m = fmaxf(m, fabsf(v[j]));  // fmaxf drops NaN operands
    }
  };
  for_each_chunk<T, kAbsmaxRowsInFlight>(p, (const T*)p.x + b * p.xs_b + h * p.xs_h, p.S, p.xs_s, take);
  if (p.S2 > 0) for_each_chunk<T, kAbsmaxRowsInFlight>(p, (const T*)p.x2 + b * p.x2s_b + h * p.x2s_h, p.S2, p.x2s_s, take);
  m = block_max(m);
  if (threadIdx.x == 0) {
    if (p.partials != nullptr) p.partials[(int64_t)bh * gridDim.x + blockIdx.x] = m;
    // non-negative floats order like their bit patterns
    else atomicMax((unsigned int*)(p.amax + (p.per_tensor ? 0 : bh)), __float_as_uint(m));
  }
}

// Scale and cast of a (batch, head) slice of both tensors.  The scale is the static one, or comes
// from the partial maxima of the abs-max pass (folded here by every workgroup; the first
// workgroup of a slice also stores the slice's descale), or from the amax buffer.
template <typename T>
__global__ __launch_bounds__(256) void cast_kernel(const QuantParams p, const int partials_per_slice) {
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh - b * p.H;
  float scale;
  if (p.scale_in != nullptr) {
    scale = *p.scale_in;
  } else if (p.partials != nullptr) {
    const int n = p.per_tensor ? partials_per_slice * (int)gridDim.y : partials_per_slice;
    const float* src = p.partials + (p.per_tensor ? 0 : (int64_t)bh * partials_per_slice);
    float am = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) am = fmaxf(am, src[i]);
    am = block_max(am);
    scale = am > 0.f ? am / kFp8Max : 1.0f;
  } else {
    const float am = p.amax[p.per_tensor ? 0 : bh];
    scale = am > 0.f ? am / kFp8Max : 1.0f;
  }
  if ((p.scale_in != nullptr || p.partials != nullptr) && blockIdx.x == 0 && threadIdx.x == 0) p.descale[bh] = scale;
  auto cast_to = [&](unsigned char* y, int64_t ys_s) {
    return [&, y, ys_s](float (&v)[8], int64_t s, int c, bool live) {
#pragma unroll
      for (int j = 0; j < 8; j++) v[j] = v[j] / scale;
      int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], w0, true);
      int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], 0, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], w1, true);
      i32x2 w = {w0, w1};
      if (live) *(i32x2*)(y + s * ys_s + c * 8) = w;
    };
  };
  for_each_chunk<T>(p, (const T*)p.x + b * p.xs_b + h * p.xs_h, p.S, p.xs_s,
                    cast_to((unsigned char*)p.y + b * p.ys_b + h * p.ys_h, p.ys_s));
  if (p.S2 > 0)
    for_each_chunk<T>(p, (const T*)p.x2 + b * p.x2s_b + h * p.x2s_h, p.S2, p.x2s_s,
                      cast_to((unsigned char*)p.y2 + b * p.y2s_b + h * p.y2s_h, p.y2s_s));
}

// amax buffer -> descale values, for all B*H entries (the path without a scratch buffer).
__global__ void finalize_kernel(const QuantParams p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  // every thread reads its source before any thread overwrites entry 0 (single workgroup launch
  // when per_tensor; otherwise each thread only touches its own entry)
  float am = p.amax[p.per_tensor ? 0 : (i < n ? i : 0)];
  __syncthreads();
  if (i >= n) return;
  p.descale[i] = am > 0.f ? am / kFp8Max : 1.0f;
}

template <typename T>
static hipError_t run(const QuantParams& p, hipStream_t stream) {
  const int BH = p.B * p.H;
  const int rpb = 256 / (p.D >> 3);
  const int64_t rows = (int64_t)p.S + p.S2;
  int per_slice = (int)((rows + rpb * 2 * quant::kRowsInFlight - 1) / (rpb * 2 * quant::kRowsInFlight));  // ~8 rows per thread
  if (per_slice < 1) per_slice = 1;
  if (per_slice > 2048) per_slice = 2048;
  dim3 grid(per_slice, BH), block(256);
  int partials_per_slice = 0;
  if (p.scale_in == nullptr) {
    int reduce_slice;
    if (p.partials != nullptr) {
      // one slot per workgroup: as many workgroups as the scratch holds slots for
      reduce_slice = (int)(p.partial_slots / BH);
      if (reduce_slice > per_slice) reduce_slice = per_slice;
      if (reduce_slice < 1) return hipErrorInvalidValue;
      partials_per_slice = reduce_slice;
    } else {
      // every workgroup ends in one atomic max on its slice's entry: keep their number near 1024,
      // same-address atomics are served one at a time
      reduce_slice = 1024 / BH;
      if (reduce_slice < 1) reduce_slice = 1;
      if (reduce_slice > per_slice) reduce_slice = per_slice;
      hipLaunchKernelGGL(fill_zero_kernel, dim3((BH + 255) / 256), dim3(256), 0, stream, p.amax, BH);
    }
    hipLaunchKernelGGL((absmax_kernel<T>), dim3(reduce_slice, BH), block, 0, stream, p);
  }
  hipLaunchKernelGGL((cast_kernel<T>), grid, block, 0, stream, p, partials_per_slice);
  if (p.scale_in == nullptr && p.partials == nullptr) {
    // per_tensor broadcasts entry 0: keep it to one workgroup so the barrier orders read/write
    if (p.per_tensor && BH > 1024) return hipErrorInvalidValue;
    const int fb = p.per_tensor ? BH : 256;
    hipLaunchKernelGGL(finalize_kernel, dim3((BH + fb - 1) / fb), dim3(fb < 64 ? 64 : fb), 0, stream, p, BH);
  }
  return hipGetLastError();
}

}  // namespace quant

hipError_t launch_fp8_quant(const QuantParams& p, int in_dtype, hipStream_t stream) {
  if (in_dtype == 0) return quant::run<__bf16>(p, stream);
  if (in_dtype == 1) return quant::run<_Float16>(p, stream);
  if (in_dtype == 2) return quant::run<float>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace xdit
