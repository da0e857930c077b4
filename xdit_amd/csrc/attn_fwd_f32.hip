// Non-causal attention forward for fp32 tensors on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32) of gfx950, any head_dim that is a multiple of 8 up to 128 (e.g. 72):
// exact fp32 products, fp32 accumulation.  (16-bit tensors of every such head_dim run on the
// 16-bit kernel.)  Same orientation as the 16-bit kernel:
//   S^T = K Q^T  (A = K rows, B = Q^T in registers),  O^T = V^T P^T  (B = P^T = the S^T registers).
// With a contraction depth of 2 per instruction every operand is ONE float per lane, so V^T is a
// plain LDS read (lanes along head_dim) and needs no transposing load.
//
// workgroup = 256 threads = 4 wavefronts x 32 query rows; K/V tiles of 32 keys, one LDS buffer,
// global loads for the next tile are held in registers while the current tile is computed.
#include "common.h"
#include "launchers.h"

namespace xdit {

namespace f32path {

constexpr int kRowsPerBlock = 128;
constexpr int kKeys = 32;

template <typename T> __device__ __forceinline__ void load8(const T* p, float (&x)[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&x)[8]) {
  f32x4 a = ((const f32x4*)p)[0], b = ((const f32x4*)p)[1];
  for (int i = 0; i < 4; i++) { x[i] = a[i]; x[4 + i] = b[i]; }
}

// D8 = head_dim / 8.  The first product contracts exactly head_dim; the second works on 32-wide
// blocks of head_dim (columns past head_dim are zero in LDS and are not stored).
template <typename T, int D8>
__global__ __launch_bounds__(256) void attn_fwd_f32_kernel(const AttnParams p) {
  constexpr int D = 8 * D8;
  constexpr int DB = (D + 31) / 32;
  constexpr int DP = 32 * DB;       // padded head_dim
  constexpr int LD = DP + 1;        // LDS row stride in floats (odd: conflict-free column reads)
  constexpr int CHUNKS = DP / 8;    // 8-element chunks per padded row
  constexpr int PER_THREAD = (kKeys * CHUNKS + 255) / 256;

  __shared__ float ks[kKeys * LD];
  __shared__ float vs[kKeys * LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const int tile = xcd_tile_index(blockIdx.x, p.tiles_per_xcd);
  if (tile >= p.total_tiles) return;
  const int bh = tile / p.nq_tiles;
  const int qt = tile - bh * p.nq_tiles;
  const int b = bh / p.H;
  const int h = bh - b * p.H;

  // Q^T fragments: lane (query l32, half hh) holds Q[query][2ks + hh] for every step ks.
  const int qrow = qt * kRowsPerBlock + wave * 32 + l32;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;
  const T* qptr = (const T*)p.q + b * p.qs_b + h * p.qs_h + (int64_t)qrow_c * p.qs_s;
  float qf[DP / 2];
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    float x[8];
    if (c * 8 < D) {
      load8<T>(qptr + c * 8, x);
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) x[i] = 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) qf[c * 4 + i] = hh ? x[2 * i + 1] : x[2 * i];
  }

  const T* kbase1 = (const T*)p.k + b * p.ks_b + h * p.ks_h;
  const T* vbase1 = (const T*)p.v + b * p.vs_b + h * p.vs_h;
  const T* kbase2 = p.Sk2 > 0 ? (const T*)p.k2 + b * p.k2s_b + h * p.k2s_h : kbase1;
  const T* vbase2 = p.Sk2 > 0 ? (const T*)p.v2 + b * p.v2s_b + h * p.v2s_h : vbase1;
  const int nt1 = (p.Sk + kKeys - 1) / kKeys;
  const int nt2 = (p.Sk2 + kKeys - 1) / kKeys;
  const int nt = nt1 + nt2;

  // staging registers: this thread's 8-element chunks of the next K and V tile
  float kreg[PER_THREAD][8], vreg[PER_THREAD][8];
  auto fetch = [&](int t) {
    const T* kb;
    const T* vb;
    int64_t kss, vss;
    int row0, valid;
    if (t < nt1) {
      kb = kbase1; vb = vbase1; kss = p.ks_s; vss = p.vs_s; row0 = t * kKeys; valid = p.Sk - row0;
    } else {
      kb = kbase2; vb = vbase2; kss = p.k2s_s; vss = p.v2s_s; row0 = (t - nt1) * kKeys; valid = p.Sk2 - row0;
    }
#pragma unroll
    for (int i = 0; i < PER_THREAD; i++) {
      const int idx = i * 256 + tid;
      const int r = idx / CHUNKS, c = idx - r * CHUNKS;
      const bool live = (idx < kKeys * CHUNKS) && (r < valid) && (c * 8 < D);
      if (live) {
        load8<T>(kb + (int64_t)(row0 + r) * kss + c * 8, kreg[i]);
        load8<T>(vb + (int64_t)(row0 + r) * vss + c * 8, vreg[i]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; j++) { kreg[i][j] = 0.f; vreg[i][j] = 0.f; }
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < PER_THREAD; i++) {
      const int idx = i * 256 + tid;
      const int r = idx / CHUNKS, c = idx - r * CHUNKS;
      if (idx < kKeys * CHUNKS) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
          ks[r * LD + c * 8 + j] = kreg[i][j];
          vs[r * LD + c * 8 + j] = vreg[i][j];
        }
      }
    }
  };

  const float c = p.scale * kLog2e;
  float m_run = -INFINITY;
  float l_part = 0.f;
  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;

  fetch(0);
  for (int t = 0; t < nt; t++) {
    __syncthreads();  // everyone is done reading the previous tile
    stage();
    __syncthreads();
    if (t + 1 < nt) fetch(t + 1);

    // S^T = K Q^T : 32 keys x 32 queries
    f32x16 sacc;
#pragma unroll
    for (int i = 0; i < 16; i++) sacc[i] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 2; s++) {
      const float kf = ks[l32 * LD + 2 * s + hh];
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf, qf[s], sacc, 0, 0, 0);
    }
    const int valid = (t < nt1) ? p.Sk - t * kKeys : p.Sk2 - (t - nt1) * kKeys;
    if (valid < kKeys) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int key = 8 * (i >> 2) + 4 * hh + (i & 3);
        if (key >= valid) sacc[i] = -INFINITY;
      }
    }
    float mx = sacc[0];
#pragma unroll
    for (int i = 1; i < 16; i++) mx = fmaxf(mx, sacc[i]);
    mx = max_halves(mx);
    const float m_new = fmaxf(m_run, mx);
    const float alpha = fast_exp2((m_run - m_new) * c);
    m_run = m_new;
    l_part *= alpha;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
    const float mc = m_run * c;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sacc[i] = exp2f(__builtin_fmaf(sacc[i], c, -mc));
      l_part += sacc[i];
    }
    // O^T += V^T P^T : register i of P^T is keys {8(i/4) + i%4, +4} for the two lane halves
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int key = 8 * (i >> 2) + 4 * hh + (i & 3);
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const float vf = vs[key * LD + 32 * db + l32];
        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf, sacc[i], oacc[db], 0, 0, 0);
      }
    }
  }

  const float l_tot = sum_halves(l_part);
  const float inv = 1.0f / l_tot;
  if (qrow < p.Sq) {
    T* optr = (T*)p.out + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_s;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int d = 32 * db + 8 * (i >> 2) + 4 * hh + (i & 3);
        if (d < D) optr[d] = (T)(oacc[db][i] * inv);
      }
    if (p.lse != nullptr && hh == 0) {
      p.lse[b * p.ls_b + h * p.ls_h + qrow] = (m_run * c + log2f(l_tot)) * kLn2;
    }
  }
}

template <typename T, int D8>
static void launch_d(const AttnParams& q, int d8, dim3 grid, hipStream_t stream) {
  if constexpr (D8 <= 16) {
    if (d8 == D8) hipLaunchKernelGGL((attn_fwd_f32_kernel<T, D8>), grid, dim3(256), 0, stream, q);
    else launch_d<T, D8 + 1>(q, d8, grid, stream);
  }
}

template <typename T>
static hipError_t launch_t(const AttnParams& q, int D, dim3 grid, hipStream_t stream) {
  if (D <= 0 || D % 8 != 0 || D > 128) return hipErrorInvalidValue;
  launch_d<T, 1>(q, D / 8, grid, stream);
  return hipGetLastError();
}

}  // namespace f32path

// Workgroups of 128 query rows: smaller ones (64 or 32 rows, to fill the chip on small problems)
// were measured and are not faster (PixArt-512 fp32, 16 x 1024 rows: 136 / 140 / 156 us): the
// number of wavefronts, each bound by its own chain of MFMAs, stays the same.
hipError_t launch_attn_fwd_f32(const AttnParams& p, int D, hipStream_t stream) {
  AttnParams q = p;
  q.nq_tiles = (p.Sq + f32path::kRowsPerBlock - 1) / f32path::kRowsPerBlock;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  dim3 grid(q.tiles_per_xcd * 8);
  return f32path::launch_t<float>(q, D, grid, stream);
}

}  // namespace xdit
