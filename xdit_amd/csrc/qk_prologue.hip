// Pre-attention prologue for gfx950: RMSNorm of Q or K + rotary embedding + head split, one pass.
//
// What an xDiT attention processor does between the QKV projections and the attention call
// (xfuser/model_executor/models/transformers/transformer_flux.py:116-147,
// transformer_hunyuan_video.py:48-83, transformer_wan.py:99-122) as separate elementwise torch
// kernels, each a full read and write of the tensor:
//     x = norm(x)              diffusers RMSNorm: x * rsqrt(mean(x^2) + eps) in fp32, rounded to
//                              the weight's 16-bit dtype, then * weight (second rounding)
//     x = apply_rotary_emb(x)  (x.float() * cos + rotate(x).float() * sin).to(x.dtype)
//     x = x.transpose(1, 2)    BSHD -> BHSD view, made contiguous later by the attention adapter
// Here: one read of x, one write of y, through arbitrary (B,H,S) element strides on both sides,
// so the BSHD projection output lands BHSD-contiguous (the layout the attention kernel streams
// fastest) and text/image streams can be written into row ranges of one joint tensor (no cat).
// Arithmetic follows the reference's rounding points: fp32 statistics, a rounding to T after the
// normalisation and after the gain, separately rounded fp32 products in the rotation (this file
// is compiled with floating-point contraction off so no product is fused into the add).
// HBM-bound: 2 * sizeof(T) bytes per element plus the cos/sin rows (shared by all heads).
#include "common.h"
#include "launchers.h"

namespace xdit {

namespace prologue {

template <typename T> struct Vec8;
template <> struct Vec8<__bf16> { typedef bf16x8 type; };
template <> struct Vec8<_Float16> { typedef f16x8 type; };

template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&x)[8]) {
  const typename Vec8<T>::type v = *(const typename Vec8<T>::type*)p;
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = (float)v[i];
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, float (&x)[8]) {
  const f32x4 a = ((const f32x4*)p)[0], b = ((const f32x4*)p)[1];
#pragma unroll
  for (int i = 0; i < 4; i++) { x[i] = a[i]; x[4 + i] = b[i]; }
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&x)[8]) {
  typename Vec8<T>::type v;
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = (T)x[i];
  *(typename Vec8<T>::type*)p = v;
}
template <>
__device__ __forceinline__ void store8<float>(float* p, const float (&x)[8]) {
  f32x4 a, b;
#pragma unroll
  for (int i = 0; i < 4; i++) { a[i] = x[i]; b[i] = x[4 + i]; }
  ((f32x4*)p)[0] = a;
  ((f32x4*)p)[1] = b;
}

// v <- T(T(v * rs) * w): the two roundings of the reference's norm.  w == nullptr: no gain.
template <typename T>
__device__ __forceinline__ void normalise8(float (&v)[8], float rs, const T* w) {
  float g[8];
  if (w != nullptr) load8<T>(w, g);
#pragma unroll
  for (int i = 0; i < 8; i++) {
    v[i] = (float)(T)(v[i] * rs);
    if (w != nullptr) v[i] = (float)(T)(v[i] * g[i]);
  }
}

// Rotation of the 8 elements a lane holds (elements 8c .. 8c+7 of a row).  c / s are the row's
// cos / sin values for these elements.  `partner` holds the elements the split-half form
// pairs them with (row elements 8c +- D/2), `upper` says which half this lane is in.
// mode 1: out[j] = x[j] cos[j] + rot[j] sin[j], rot = (-x[2i+1], x[2i]) per pair  (diffusers
//         apply_rotary_emb, use_real_unbind_dim = -1)
// mode 2: rot = (-x[j + D/2]) for the lower half, x[j - D/2] for the upper (use_real_unbind_dim = -2)
// mode 3: out[2i] = x[2i] cos[2i] - x[2i+1] sin[2i+1], out[2i+1] = x[2i] sin[2i+1] + x[2i+1] cos[2i]
//         (transformer_wan.py:108-120)
__device__ __forceinline__ void rotate8(float (&v)[8], const float (&c)[8], const float (&s)[8], int mode,
                                        const float (&partner)[8], bool upper) {
  float o[8];
  if (mode == 1) {
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      o[i] = v[i] * c[i] + (-v[i + 1]) * s[i];
      o[i + 1] = v[i + 1] * c[i + 1] + v[i] * s[i + 1];
    }
  } else if (mode == 2) {
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = v[i] * c[i] + (upper ? partner[i] : -partner[i]) * s[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      o[i] = v[i] * c[i] - v[i + 1] * s[i + 1];
      o[i + 1] = v[i] * s[i + 1] + v[i + 1] * c[i];
    }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = o[i];
}

// Sum over the `lpr` consecutive lanes that hold one row (lpr a power of two, rows aligned).
// 8 and 16 lanes stay within a DPP row: two quad permutes, then the half-row and row mirrors.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false);
  return x + __builtin_bit_cast(float, y);
}
__device__ __forceinline__ float row_sum(float x, int lpr) {
  if (lpr == 16 || lpr == 8) {
    x = dpp_add<0xB1>(x);   // quad_perm [1,0,3,2]: lane ^ 1
    x = dpp_add<0x4E>(x);   // quad_perm [2,3,0,1]: lane ^ 2
    x = dpp_add<0x141>(x);  // row_half_mirror: the other quad of each 8 lanes
    if (lpr == 16) x = dpp_add<0x140>(x);  // row_mirror: the other half of each 16 lanes
    return x;
  }
  for (int m = 1; m < lpr; m <<= 1) x += __shfl_xor(x, m);
  return x;
}

// Per-head form: one wavefront per token (b, s).  A row (b, s, h) of D elements is held by `lpr`
// consecutive lanes (a power of two; lanes with 8c >= D idle), so a wavefront instruction covers
// 64/lpr adjacent heads (1 KiB of contiguous BSHD input at head_dim 128) and the wavefront walks
// over the heads of its token.  The token's cos/sin chunk and the gain chunk are loaded once per
// lane and reused for every head; kRowsInFlight rows are loaded before the first is used.
constexpr int kRowsInFlight = 4;

template <typename T>
__device__ __forceinline__ void prologue_rows(const PrologueParams& p) {
  const int64_t tok = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  if (tok >= (int64_t)p.B * p.S) return;  // whole wavefronts leave together
  const int lane = threadIdx.x & 63;
  const int c = lane & (p.lpr - 1);
  const int slot = lane / p.lpr;
  const int slots = 64 / p.lpr;
  const bool chunk_live = c * 8 < p.D;
  const int cc = chunk_live ? c : 0;  // idle lanes read chunk 0 and store nothing
  const int s = (int)(tok % p.S);
  const int b = (int)(tok / p.S);
  const T* x = (const T*)p.x + b * p.xs_b + (int64_t)s * p.xs_s + cc * 8;
  T* y = (T*)p.y + b * p.ys_b + (int64_t)s * p.ys_s + cc * 8;
  const int sr = s - p.rope_row0;
  const bool rope = p.rope_mode != 0 && sr >= 0 && sr < p.rope_rows;
  float cs[8], sn[8], g[8];
  if (rope) {
    const int64_t off = (int64_t)sr * p.rope_stride + cc * 8;
    load8<float>(p.cos + off, cs);
    load8<float>(p.sin + off, sn);
  }
  const bool gain = p.norm != 0 && p.weight != nullptr;
  if (gain) load8<T>((const T*)p.weight + cc * 8, g);
  const bool upper = (c & (p.lpr >> 1)) != 0;
  for (int h0 = 0; h0 < p.H; h0 += slots * kRowsInFlight) {  // uniform trip count
    float v[kRowsInFlight][8];
#pragma unroll
    for (int u = 0; u < kRowsInFlight; u++) {
      const int h = h0 + u * slots + slot;
      load8<T>(x + (int64_t)(h < p.H ? h : p.H - 1) * p.xs_h, v[u]);
    }
#pragma unroll
    for (int u = 0; u < kRowsInFlight; u++) {
      const int h = h0 + u * slots + slot;
      if (h0 + u * slots >= p.H) break;  // uniform
      if (p.norm) {
        float ss = 0.f;
        if (chunk_live) {
#pragma unroll
          for (int i = 0; i < 8; i++) ss += v[u][i] * v[u][i];
        }
        ss = row_sum(ss, p.lpr);
        const float rs = 1.0f / sqrtf(ss * p.inv_n + p.eps);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          v[u][i] = (float)(T)(v[u][i] * rs);
          if (gain) v[u][i] = (float)(T)(v[u][i] * g[i]);
        }
      }
      if (p.rope_mode != 0) {  // uniform: every lane takes part in the exchange below
        float partner[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (p.rope_mode == 2) {
#pragma unroll
          for (int i = 0; i < 8; i++) partner[i] = __shfl_xor(v[u][i], p.lpr >> 1);
        }
        if (rope) {
          rotate8(v[u], cs, sn, p.rope_mode, partner, upper);
#pragma unroll
          for (int i = 0; i < 8; i++) v[u][i] = (float)(T)v[u][i];
        }
      }
      if (chunk_live && h < p.H) store8<T>(y + (int64_t)h * p.ys_h, v[u]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void prologue_rows_kernel(const PrologueParams p) {
  prologue_rows<T>(p);
}

// Several tensors in one launch (the Q, K and V of the text and image streams of one attention
// block): blockIdx.y selects the job, workgroups beyond a job's tokens leave at once.
template <typename T>
__global__ __launch_bounds__(256) void prologue_rows_batch_kernel(const PrologueBatch b) {
  prologue_rows<T>(b.job[blockIdx.y]);
}

// Across-heads form (the norm statistic runs over all H*D elements of a token and the gain has
// H*D entries: Wan's norm_q / norm_k, transformer_wan.py:99-100): one workgroup per token, up to
// kChunks 8-element chunks per thread held in registers between the reduction and the store.
constexpr int kChunks = 4;

template <typename T>
__global__ __launch_bounds__(256) void prologue_token_kernel(const PrologueParams p) {
  const int64_t tok = blockIdx.x;
  const int s = (int)(tok % p.S);
  const int b = (int)(tok / p.S);
  const int cpr = p.D >> 3;
  const int chunks = p.H * cpr;
  float v[kChunks][8] = {};
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kChunks; k++) {
    const int j = threadIdx.x + 256 * k;
    if (j < chunks) {
      const int h = j / cpr, c = j - h * cpr;
      load8<T>((const T*)p.x + b * p.xs_b + h * p.xs_h + (int64_t)s * p.xs_s + c * 8, v[k]);
#pragma unroll
      for (int i = 0; i < 8; i++) ss += v[k][i] * v[k][i];
    }
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) ss += __shfl_xor(ss, m);
  __shared__ float part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float rs = 1.0f / sqrtf((part[0] + part[1] + part[2] + part[3]) * p.inv_n + p.eps);
  const int sr = s - p.rope_row0;
  const bool rope = p.rope_mode != 0 && sr >= 0 && sr < p.rope_rows;
  float cs[8], sn[8];
  if (rope) {  // cpr divides 256: a thread's chunks all sit at the same place c of their rows
    const int64_t off = (int64_t)sr * p.rope_stride + (threadIdx.x & (cpr - 1)) * 8;
    load8<float>(p.cos + off, cs);
    load8<float>(p.sin + off, sn);
  }
#pragma unroll
  for (int k = 0; k < kChunks; k++) {
    const int j = threadIdx.x + 256 * k;
    const bool live = j < chunks;  // chunks is a multiple of cpr and cpr divides 64: a row's lanes are live together
    const int h = live ? j / cpr : 0, c = live ? j - h * cpr : 0;
    if (live) normalise8<T>(v[k], rs, p.weight != nullptr ? (const T*)p.weight + (int64_t)h * p.D + c * 8 : (const T*)nullptr);
    float partner[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (p.rope_mode == 2) {
#pragma unroll
      for (int i = 0; i < 8; i++) partner[i] = __shfl_xor(v[k][i], cpr >> 1);
    }
    if (live && rope) {
      rotate8(v[k], cs, sn, p.rope_mode, partner, (c & (cpr >> 1)) != 0);
#pragma unroll
      for (int i = 0; i < 8; i++) v[k][i] = (float)(T)v[k][i];
    }
    if (live) store8<T>((T*)p.y + b * p.ys_b + h * p.ys_h + (int64_t)s * p.ys_s + c * 8, v[k]);
  }
}

template <typename T>
static hipError_t run(const PrologueParams& p, hipStream_t stream) {
  if (p.norm == 2) {
    hipLaunchKernelGGL((prologue_token_kernel<T>), dim3((unsigned)((int64_t)p.B * p.S)), dim3(256), 0, stream, p);
  } else {
    const int64_t tokens = (int64_t)p.B * p.S;  // one wavefront each, four per workgroup
    hipLaunchKernelGGL((prologue_rows_kernel<T>), dim3((unsigned)((tokens + 3) / 4)), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

template <typename T>
static hipError_t run_batch(const PrologueBatch& b, hipStream_t stream) {
  int64_t tokens = 0;
  for (int i = 0; i < b.n; i++) {
    const int64_t t = (int64_t)b.job[i].B * b.job[i].S;
    if (t > tokens) tokens = t;
  }
  hipLaunchKernelGGL((prologue_rows_batch_kernel<T>), dim3((unsigned)((tokens + 3) / 4), (unsigned)b.n), dim3(256), 0, stream, b);
  return hipGetLastError();
}

}  // namespace prologue

hipError_t launch_qk_prologue_batch(const PrologueBatch& b, int dtype, hipStream_t stream) {
  if (dtype == 0) return prologue::run_batch<__bf16>(b, stream);
  if (dtype == 1) return prologue::run_batch<_Float16>(b, stream);
  if (dtype == 2) return prologue::run_batch<float>(b, stream);
  return hipErrorInvalidValue;
}

int prologue_max_token_elems() { return prologue::kChunks * 256 * 8; }

hipError_t launch_qk_prologue(const PrologueParams& p, int dtype, hipStream_t stream) {
  if (dtype == 0) return prologue::run<__bf16>(p, stream);
  if (dtype == 1) return prologue::run<_Float16>(p, stream);
  if (dtype == 2) return prologue::run<float>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace xdit
