// Non-causal attention forward for fp32 tensors on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32) of gfx950, any head_dim that is a multiple of 8 up to 128 (e.g. 72):
// exact fp32 products, fp32 accumulation.  (16-bit tensors of every such head_dim run on the
// 16-bit kernel.)  Same orientation as the 16-bit kernel:
//   S^T = K Q^T  (A = K rows, B = Q^T in registers),  O^T = V^T P^T  (B = P^T = the S^T registers).
// With a contraction depth of 2 per instruction every operand is ONE float per lane, so V^T is a
// plain LDS read (lanes along head_dim) and needs no transposing load.
//
// workgroup = 256 threads = 4 wavefronts, each with 32 query rows and 32 of the keys of a tile.
// KS = 1: four row groups (128 query rows) share tiles of 32 keys.  KS = 2: two row groups (64
// query rows), and the two wavefronts of a row group each take one half of every 64-key tile and
// fold their partial results through LDS at the end: twice the workgroups and wavefronts, for
// problems whose 128-row tiles would leave compute units idle (PixArt-512: 16 heads x 1024 rows
// are 128 such tiles for 256 compute units).  Every wavefront is bound by its own chain of MFMAs
// (64 cycles each), so what counts is how many SIMDs have one.
//
// K/V tiles are double buffered in LDS and filled by direct global->LDS loads (16 bytes per lane,
// one barrier per tile).  A tile is an array of 16-byte chunks in the order the loads write them:
// K rows of DP/4 + 1 chunks, V rows of DP/4 + 2 chunks (DP = head_dim rounded up to 32); the
// lanes of the chunks a row does not have stay idle.  The K pitch of DP + 4 floats makes the
// 16-byte fragment reads of 16 consecutive rows hit 64 different banks; the V pitch of DP + 8
// floats puts the rows that the two halves of a wavefront read (4 keys apart) 32 banks apart.
//
// The contraction index of the first product is permuted so that a lane's K operands of four
// consecutive steps are 16 contiguous bytes: step s of lane half hh is column 8(s/4) + 4hh + s%4.
#include "attn_split.h"
#include "launchers.h"

namespace xdit {

namespace f32path {

template <int D8, int KS> struct Geom {
  static constexpr int D = 8 * D8;
  static constexpr int DB = (D + 31) / 32;
  static constexpr int DP = 32 * DB;   // padded head_dim of the second product
  static constexpr int KCH = DP / 4 + 1;   // 16-byte chunks per K row in LDS
  static constexpr int VCH = DP / 4 + 2;   // ... per V row
  static constexpr int TK = 32 * KS;       // keys per tile
  static constexpr int RQ = 4 / KS;        // row groups (of 32 query rows) per workgroup
  static constexpr int ROWS = 32 * RQ;
  static constexpr int K_CHUNKS = TK * KCH;
  static constexpr int V_CHUNKS = TK * VCH;
  static constexpr int K_INSTR = (K_CHUNKS + 63) / 64;   // wavefront load instructions per K tile
  static constexpr int V_INSTR = (V_CHUNKS + 63) / 64;
  static constexpr int K_BYTES = K_INSTR * 1024;
  static constexpr int V_BYTES = V_INSTR * 1024;
  static constexpr int BUF_BYTES = K_BYTES + V_BYTES;
  // partial result of a wavefront for the fold between key halves: 16 DB + 2 floats per lane
  static constexpr int PART_BYTES = (16 * DB + 2) * 64 * 4;
  static constexpr int LDS_BYTES = 2 * BUF_BYTES > RQ * PART_BYTES ? 2 * BUF_BYTES : RQ * PART_BYTES;
};

// FUSED: the ring step; the block is folded into the fp32 accumulator (p.acc_out, p.acc_lse) with
// the arithmetic of the merge kernel instead of being written out.
template <int D8, int KS, bool FUSED>
__global__ __launch_bounds__(256) void attn_fwd_f32_kernel(const AttnParams p) {
  typedef Geom<D8, KS> G;
  constexpr int D = G::D, DB = G::DB, TK = G::TK, RQ = G::RQ;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hh = lane >> 5;
  const int rg = wave % RQ;    // row group of this wavefront
  const int ksl = wave / RQ;   // which 32 keys of a tile it takes

  const int tile = xcd_tile_index(blockIdx.x, p.tiles_per_xcd);
  if (tile >= p.total_tiles) return;
  const int bh = tile / p.nq_tiles;
  const int qt = tile - bh * p.nq_tiles;
  const int b = bh / p.H;
  const int h = bh - b * p.H;

  // Q^T fragments: lane (query l32, half hh) holds Q[query][8j + 4hh + i] as step 4j + i.
  const int qrow = qt * G::ROWS + rg * 32 + l32;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;
  const float* qptr = (const float*)p.q + b * p.qs_b + h * p.qs_h + (int64_t)qrow_c * p.qs_s + 4 * hh;
  f32x4 qf[D8];
#pragma unroll
  for (int j = 0; j < D8; j++) qf[j] = *(const f32x4*)(qptr + 8 * j);

  const unsigned char* kbase1 = (const unsigned char*)((const float*)p.k + b * p.ks_b + h * p.ks_h);
  const unsigned char* vbase1 = (const unsigned char*)((const float*)p.v + b * p.vs_b + h * p.vs_h);
  const unsigned char* kbase2 = p.Sk2 > 0 ? (const unsigned char*)((const float*)p.k2 + b * p.k2s_b + h * p.k2s_h) : kbase1;
  const unsigned char* vbase2 = p.Sk2 > 0 ? (const unsigned char*)((const float*)p.v2 + b * p.v2s_b + h * p.v2s_h) : vbase1;
  const unsigned kss1 = (unsigned)p.ks_s * 4, vss1 = (unsigned)p.vs_s * 4;
  const unsigned kss2 = p.Sk2 > 0 ? (unsigned)p.k2s_s * 4 : kss1, vss2 = p.Sk2 > 0 ? (unsigned)p.v2s_s * 4 : vss1;
  const int nt1 = (p.Sk + TK - 1) / TK;
  const int nt = nt1 + (p.Sk2 + TK - 1) / TK;
  const unsigned lds_base = (unsigned)(uintptr_t)(XDIT_LDS unsigned char*)smem;

  // Loads KV tile t into buffer `buf`: load instruction n of a tile (n = wave, wave + 4, ...)
  // writes chunks 64n .. 64n+63; chunk x is row x / CH, 16-byte column x % CH.  Rows past the end
  // of a KV segment re-read its last row (their logits are masked, their P is exactly zero).
  auto issue_tile = [&](int t, int buf) {
    const bool second = t >= nt1;
    const unsigned row0 = (unsigned)(second ? t - nt1 : t) * TK;
    const unsigned kss = second ? kss2 : kss1, vss = second ? vss2 : vss1;
    const unsigned char* kp = (second ? kbase2 : kbase1) + (uint64_t)row0 * kss;
    const unsigned char* vp = (second ? vbase2 : vbase1) + (uint64_t)row0 * vss;
    const int left = (second ? p.Sk2 : p.Sk) - (int)row0;
    const int last = (left < TK ? left : TK) - 1;
    const unsigned bo = lds_base + buf * G::BUF_BYTES;
#pragma unroll
    for (int n = 0; n < (G::K_INSTR + 3) / 4; n++) {
      const int instr = 4 * n + wave;
      const int x = instr * 64 + lane;
      int r = x / G::KCH;
      const int cchunk = x - r * G::KCH;
      r = r < last ? r : last;
      if (instr < G::K_INSTR && x < G::K_CHUNKS && cchunk < D / 4)
        load_lds_16(kp, (unsigned)r * kss + cchunk * 16, bo + instr * 1024);
    }
#pragma unroll
    for (int n = 0; n < (G::V_INSTR + 3) / 4; n++) {
      const int instr = 4 * n + wave;
      const int x = instr * 64 + lane;
      int r = x / G::VCH;
      const int cchunk = x - r * G::VCH;
      r = r < last ? r : last;
      if (instr < G::V_INSTR && x < G::V_CHUNKS && cchunk < D / 4)
        load_lds_16(vp, (unsigned)r * vss + cchunk * 16, bo + G::K_BYTES + instr * 1024);
    }
  };

  const float c = p.scale * kLog2e;
  float m_used = -INFINITY;   // running (lazily updated) row maximum of the raw dot products
  float l_part = 0.f;
  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;

  issue_tile(0, 0);
  for (int t = 0; t < nt; t++) {
    const int buf = t & 1;
    // tile t has landed (this thread's loads, after the barrier everyone's), and every wavefront
    // is done reading the other buffer, which the next tile now overwrites
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 1 < nt) issue_tile(t + 1, buf ^ 1);

    const int valid = ((t < nt1) ? p.Sk - t * TK : p.Sk2 - (t - nt1) * TK) - 32 * ksl;  // keys of this wavefront's slice
    if (valid <= 0) continue;
    const XDIT_LDS unsigned char* kt = (const XDIT_LDS unsigned char*)smem + buf * G::BUF_BYTES;
    const XDIT_LDS unsigned char* vt = kt + G::K_BYTES;

    // S^T = K Q^T : 32 keys x 32 queries
    f32x16 sacc;
#pragma unroll
    for (int i = 0; i < 16; i++) sacc[i] = 0.f;
    const XDIT_LDS unsigned char* krow = kt + ((32 * ksl + l32) * G::KCH + hh) * 16;
#pragma unroll
    for (int j = 0; j < D8; j++) {
      const f32x4 kf = *(const XDIT_LDS f32x4*)(krow + 32 * j);
#pragma unroll
      for (int i = 0; i < 4; i++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[i], qf[j][i], sacc, 0, 0, 0);
    }
    if (valid < 32) {
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
    const float m_new = fmaxf(m_used, mx);
    const bool grow = (m_new - m_used) * c > kLazyRescaleLog2;  // true on the first tile (-inf)
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float alpha = fast_exp2((m_used - m_new) * c);  // 0 on the first tile
      m_used = m_new;
      l_part *= alpha;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
    }
    const float mc = m_used * c;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sacc[i] = exp2f(__builtin_fmaf(sacc[i], c, -mc));
      l_part += sacc[i];
    }
    // O^T += V^T P^T : register i of P^T is keys {8(i/4) + i%4, +4} for the two lane halves
    const XDIT_LDS float* vcol = (const XDIT_LDS float*)(vt + (32 * ksl + 4 * hh) * G::VCH * 16) + l32;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int key = 8 * (i >> 2) + (i & 3);
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const float vf = vcol[key * G::VCH * 4 + 32 * db];
        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf, sacc[i], oacc[db], 0, 0, 0);
      }
    }
  }

  if constexpr (KS > 1) {
    // fold the partial results of the key halves of a row group: the wavefronts of the second half
    // leave theirs in LDS ([value][lane], so that lanes write and read consecutive floats)
    __syncthreads();  // the tile buffers are no longer read
    XDIT_LDS float* part = (XDIT_LDS float*)smem + rg * (G::PART_BYTES / 4) + lane;
    if (ksl != 0) {
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) part[(16 * db + i) * 64] = oacc[db][i];
      part[16 * DB * 64] = m_used;
      part[(16 * DB + 1) * 64] = l_part;
    }
    __syncthreads();
    if (ksl != 0) return;
    const float m1 = part[16 * DB * 64], l1 = part[(16 * DB + 1) * 64];
    const float m = fmaxf(m_used, m1);   // m_used is finite: the first half of tile 0 holds key 0
    const float a0 = fast_exp2((m_used - m) * c), a1 = fast_exp2((m1 - m) * c);  // a1 = 0 for a half that saw no key
    m_used = m;
    l_part = l_part * a0 + l1 * a1;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] = oacc[db][i] * a0 + part[(16 * db + i) * 64] * a1;
  }

  const float l_tot = sum_halves(l_part);
  const float inv = 1.0f / l_tot;
  const float lse = (m_used * c + log2f(l_tot)) * kLn2;
  if (qrow >= p.Sq) return;
  if constexpr (!FUSED) {
    float* optr = (float*)p.out + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_s;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        const int d = 32 * db + 8 * a + 4 * hh;   // registers 4a..4a+3 are d .. d+3 of this lane's query
        if (d < D) {
          const f32x4 o = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv, oacc[db][4 * a + 3] * inv};
          *(f32x4*)(optr + d) = o;
        }
      }
    if (p.lse != nullptr && hh == 0) p.lse[b * p.ls_b + h * p.ls_h + qrow] = lse;
  } else {
    // ring step: the arithmetic of the merge kernel on this block (fp32, so nothing is rounded in
    // between); both halves of the wavefront read the row's log-sum-exp before one of them
    // overwrites it (program order within the wavefront)
    const bool first = p.acc_first != 0;
    float* alp = p.acc_lse + b * p.al_b + h * p.al_h + (int64_t)qrow * p.al_s;
    float w = 0.f, new_lse = lse;
    if (!first) {
      const float la = *alp;
      w = sigmoid(lse - la);
      new_lse = la - log_sigmoid(la - lse);
    }
    float* aptr = p.acc_out + b * p.ao_b + h * p.ao_h + (int64_t)qrow * p.ao_s;
    float* optr = p.out != nullptr ? (float*)p.out + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_s : nullptr;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        const int d = 32 * db + 8 * a + 4 * hh;
        if (d < D) {
          f32x4 m = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv, oacc[db][4 * a + 3] * inv};
          if (!first) {
            const f32x4 acc = *(const f32x4*)(aptr + d);
#pragma unroll
            for (int e = 0; e < 4; e++) m[e] = fold_value(acc[e], m[e], w);
          }
          if (p.acc_store) *(f32x4*)(aptr + d) = m;
          if (optr != nullptr) *(f32x4*)(optr + d) = m;
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (hh == 0) {
      *alp = new_lse;
      if (p.lse != nullptr) p.lse[b * p.ls_b + h * p.ls_h + qrow] = new_lse;
    }
  }
}

template <int D8, int KS, bool FUSED>
static hipError_t launch_kernel(const AttnParams& q, dim3 grid, hipStream_t stream) {
  typedef Geom<D8, KS> G;
  static std::atomic<bool> lds_ready[kMaxDevices];
  const int slot = current_device_slot();
  if (G::LDS_BYTES > 65536 && !lds_ready[slot].load(std::memory_order_relaxed)) {  // > 64 KiB of dynamic LDS must be enabled once per kernel and device
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_f32_kernel<D8, KS, FUSED>, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
    if (e != hipSuccess) return e;
    lds_ready[slot].store(true, std::memory_order_relaxed);
  }
  hipLaunchKernelGGL((attn_fwd_f32_kernel<D8, KS, FUSED>), grid, dim3(256), G::LDS_BYTES, stream, q);
  return hipGetLastError();
}

template <int D8, int KS, bool FUSED>
static hipError_t launch_d(const AttnParams& q, int d8, dim3 grid, hipStream_t stream) {
  if constexpr (D8 <= 16) {
    if (d8 == D8) return launch_kernel<D8, KS, FUSED>(q, grid, stream);
    return launch_d<D8 + 1, KS, FUSED>(q, d8, grid, stream);
  } else {
    return hipErrorInvalidValue;
  }
}

}  // namespace f32path

// Query rows per workgroup: 128, or 64 with the keys of a tile split between two wavefronts when
// 128-row tiles would leave more than a quarter of the compute units without a workgroup.
// (Smaller workgroups without the key split were measured and do not help: PixArt-512 fp32,
// 16 x 1024 rows: 136 / 140 / 156 us at 128 / 64 / 32 rows, since the number of wavefronts, each
// bound by its own chain of MFMAs, stays the same.)
int attn_fwd_f32_rows(const AttnParams& p) {
  const int64_t tiles128 = (int64_t)p.B * p.H * ((p.Sq + 127) / 128);
  return tiles128 * 4 < (int64_t)resident_cus(p.cu_count) * 3 ? 64 : 128;
}

hipError_t launch_attn_fwd_f32(const AttnParams& p, int D, hipStream_t stream) {
  if (D <= 0 || D % 8 != 0 || D > 128) return hipErrorInvalidValue;
  AttnParams q = p;
  const int rows = attn_fwd_f32_rows(p);
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  dim3 grid(q.tiles_per_xcd * 8);
  const bool fused = p.acc_out != nullptr;
  if (rows == 64) return fused ? f32path::launch_d<1, 2, true>(q, D / 8, grid, stream) : f32path::launch_d<1, 2, false>(q, D / 8, grid, stream);
  return fused ? f32path::launch_d<1, 1, true>(q, D / 8, grid, stream) : f32path::launch_d<1, 1, false>(q, D / 8, grid, stream);
}

}  // namespace xdit
