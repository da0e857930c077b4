// Non-causal attention forward for fp8 (OCP e4m3fn) Q/K/V with per-(batch, head) fp32 descales,
// head_dim 128, bf16 or fp16 output, fp32 log-sum-exp, on gfx950.
//
// Same structure as the 16-bit kernel (workgroup = 4, 8 or 12 wavefronts x 32 query rows, 64-key
// K/V tiles double buffered in LDS by direct global->LDS loads, hand-issued LDS fragment reads,
// transposed products so that each lane owns one query), with v_mfma_f32_32x32x64_f8f6f4 for both products:
//   S^T = K Q^T    A = K rows, B = Q^T (registers); contraction over head_dim, 64 per instruction.
//                  A and B use the same lane->contraction-index map, so each lane simply holds the
//                  32 contiguous bytes d = 64ks + 32(l/32) .. +31 of its row.
//   O^T = V^T P^T  contraction over the 64 keys of the tile in ONE instruction per 32 rows of
//                  head_dim.  P^T is the S^T accumulator converted to fp8 in register order, so
//                  byte e = 16kb + i of lane (query, half hh) is key 32kb + 8(i/4) + 4hh + i%4;
//                  V^T is fetched with ds_read_b64_tr_b8, whose source lanes are pointed at exactly
//                  those key rows, so both operands agree on the byte -> key map.
// P is scaled by 2^kPShift before the fp8 conversion so the bulk of the probabilities sits in
// e4m3's normal range; the same factor is in the row sum, so it cancels in the output and is
// subtracted from the log-sum-exp.  Logits are (q.k) * softmax_scale * q_descale * k_descale; the
// output is multiplied by v_descale.
#include "attn_split.h"
#include "launchers.h"

namespace xdit {

namespace fp8path {

constexpr int kRowsPerWave = 32;
constexpr int D = 128;
constexpr float kPShift = 6.0f;           // P is scaled by 2^6 ...
constexpr float kLazyRescaleLog2 = 2.0f;  // ... and the row max may lag by 2^2: P <= 2^8 < 448

// LDS tile geometry: rows of 128 bytes, 8 rows per 1 KiB piece, 8 pieces per 64-key tile;
// row r lives in piece r % 8 at slot r / 8.  Piece pitches pad by 16 B (K: 16-byte reads of 16
// consecutive rows) and 32 B (V: 32-byte row segments of 8 rows) to spread the banks.
constexpr int ROW_BYTES = 128;
constexpr int NG = 8;
constexpr int K_PITCH = 1024 + 16;
constexpr int V_PITCH = 1024 + 32;
constexpr int K_BYTES = NG * K_PITCH;
constexpr int V_BYTES = NG * V_PITCH;
constexpr int BUF_BYTES = K_BYTES + V_BYTES;
// LDS fragment reads are issued this many MFMAs ahead of the MFMA that consumes them.
constexpr int kPrefetch = 2;

// One segment of work: query tile `tile`, KV tiles [it0, it1); see attn_split.h for part_out.
template <typename TO, int NW>
__device__ __forceinline__ void attn_segment_fp8(const AttnParams& p, unsigned char* smem, const int tile,
                                                 const int it0, const int it1, TO* part_out, float* part_lse) {
  typedef unsigned char u8;
  constexpr int kWaves = NW;
  constexpr int kRowsPerBlock = kRowsPerWave * kWaves;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const int bh = tile / p.nq_tiles;
  const int qt = tile - bh * p.nq_tiles;
  const int b = bh / p.H;
  const int h = bh - b * p.H;

  // ---- Q fragments: 2 contraction steps x 32 bytes ---------------------------------------
  const int qrow = qt * kRowsPerBlock + wave * kRowsPerWave + l32;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;
  const u8* qptr = (const u8*)p.q + b * p.qs_b + h * p.qs_h + (int64_t)qrow_c * p.qs_s + hh * 32;
  i32x8 qf[2];
#pragma unroll
  for (int ks = 0; ks < 2; ks++) {
    i32x4 lo = *(const i32x4*)(qptr + ks * 64);
    i32x4 hi = *(const i32x4*)(qptr + ks * 64 + 16);
    qf[ks] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }

  // ---- tile loads ------------------------------------------------------------------------
  const u8* kbase1 = (const u8*)p.k + b * p.ks_b + h * p.ks_h;
  const u8* vbase1 = (const u8*)p.v + b * p.vs_b + h * p.vs_h;
  const u8* kbase2 = p.Sk2 > 0 ? (const u8*)p.k2 + b * p.k2s_b + h * p.k2s_h : kbase1;
  const u8* vbase2 = p.Sk2 > 0 ? (const u8*)p.v2 + b * p.v2s_b + h * p.v2s_h : vbase1;
  // Loader wavefronts: the first LW wavefronts each load PAIRS (K piece g, V piece g) pairs,
  // g = wave + LW * i, with one row index per lane for both pieces of a pair.
  constexpr int LW = kWaves < 8 ? kWaves : 8;
  constexpr int PAIRS = NG / LW;
  const int ld_row0 = NG * (lane >> 3) + wave;    // 8 lanes per 128-byte row: row of this lane in pair 0
  const unsigned ld_colb = (lane & 7) * 16;
  const unsigned lds_base = (unsigned)(uintptr_t)(XDIT_LDS u8*)smem;
  const unsigned ld_kdst = lds_base + wave * K_PITCH;  // LDS address of K piece `wave`, buffer 0
  const unsigned ld_vdst = lds_base + K_BYTES + wave * V_PITCH;
  const int nt1 = (p.Sk + kKeysPerTile - 1) / kKeysPerTile;

  // Stream position: base pointers of the next tile to load, byte strides, keys left in its segment.
  const u8* ld_kp;
  const u8* ld_vp;
  unsigned ld_kss, ld_vss;
  int64_t ld_kstep, ld_vstep;
  int ld_left;
  auto seek_tile = [&](int t) {
    if (t < nt1) {
      ld_kp = kbase1 + (int64_t)t * kKeysPerTile * p.ks_s;
      ld_vp = vbase1 + (int64_t)t * kKeysPerTile * p.vs_s;
      ld_kss = (unsigned)p.ks_s; ld_vss = (unsigned)p.vs_s;
      ld_kstep = kKeysPerTile * p.ks_s; ld_vstep = kKeysPerTile * p.vs_s;
      ld_left = p.Sk - t * kKeysPerTile;
    } else {
      ld_kp = kbase2 + (int64_t)(t - nt1) * kKeysPerTile * p.k2s_s;
      ld_vp = vbase2 + (int64_t)(t - nt1) * kKeysPerTile * p.v2s_s;
      ld_kss = (unsigned)p.k2s_s; ld_vss = (unsigned)p.v2s_s;
      ld_kstep = kKeysPerTile * p.k2s_s; ld_vstep = kKeysPerTile * p.v2s_s;
      ld_left = p.Sk2 - (t - nt1) * kKeysPerTile;
    }
  };
  // Loads the tile at the stream position into buffer `buf` and advances the position.
  auto issue_tile = [&](int t, int buf) {
    if (kWaves == LW || wave < LW) {
      const int last = (ld_left < kKeysPerTile ? ld_left : kKeysPerTile) - 1;
      const unsigned bo = buf * BUF_BYTES;
#pragma unroll
      for (int i = 0; i < PAIRS; i++) {
        int r = ld_row0 + LW * i;
        r = r < last ? r : last;  // rows past the end of the segment re-read its last row
        load_lds_16(ld_kp, __umul24((unsigned)r, ld_kss) + ld_colb, ld_kdst + bo + i * LW * K_PITCH);
        load_lds_16(ld_vp, __umul24((unsigned)r, ld_vss) + ld_colb, ld_vdst + bo + i * LW * V_PITCH);
      }
    }
    if (t + 1 == nt1) {
      seek_tile(t + 1);
    } else {
      ld_kp += ld_kstep; ld_vp += ld_vstep; ld_left -= kKeysPerTile;
    }
  };

  // ---- LDS read bases ------------------------------------------------------------------------
  // K fragment for key block kb, step ks: row 32kb + l32, bytes 64ks + 32hh .. +31.
  const int kbase_off = (l32 & 7) * K_PITCH + (l32 >> 3) * ROW_BYTES + hh * 32;
  // V^T fragment, read r (0..3), d block db: as a SOURCE lane of ds_read_b64_tr_b8, lane
  // (group g = lane/16, s = lane%16) supplies 8 bytes of key row 16r + 8(s/8) + 4hh + (s/2)%4
  // at d = 32db + 16(g%2) + 8(s%2); lane (g, i) receives d = 32db + 16(g%2) + i for the 8 keys
  // 16r + 8(j/4) + 4hh + j%4, j = 0..7.
  const int s16 = lane & 15;
  const int vbase_off = (4 * hh + ((s16 >> 1) & 3)) * V_PITCH + (s16 >> 3) * ROW_BYTES +
                        16 * ((lane >> 4) & 1) + 8 * (s16 & 1);

  // ---- softmax state -------------------------------------------------------------------------
  float sq = 1.f, sk = 1.f, sv = 1.f;
  if (p.q_descale) sq = p.q_descale[b * p.ds_b + h * p.ds_h];
  if (p.k_descale) sk = p.k_descale[b * p.ds_b + h * p.ds_h];
  if (p.v_descale) sv = p.v_descale[b * p.ds_b + h * p.ds_h];
  const float c = p.scale * sq * sk * kLog2e;
  float m_used = -INFINITY;
  float l_part = 0.f;
  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;

  seek_tile(it0);
  issue_tile(it0, 0);
#pragma unroll
  for (int ks = 0; ks < 2; ks++) asm volatile("" : "+v"(qf[ks]));

  for (int t = it0; t < it1; t++) {
    const int buf = (t - it0) & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t + 1 < it1) issue_tile(t + 1, buf ^ 1);

    const XDIT_LDS u8* ktile = (const XDIT_LDS u8*)(smem + buf * BUF_BYTES) + kbase_off;
    const XDIT_LDS u8* vtile = (const XDIT_LDS u8*)(smem + buf * BUF_BYTES + K_BYTES) + vbase_off;

    // ---- S^T = K Q^T ---------------------------------------------------------------------
    // Four MFMAs; MFMA m = 2 kb + ks takes the 32 bytes of its K row as two 16-byte reads.
    f32x16 sacc[2];
    {
      constexpr int PD = kPrefetch;  // MFMAs whose two reads are in flight
      constexpr int NM = 4;
      const unsigned kaddr = (unsigned)(uintptr_t)ktile;
      i32x4 klo[NM], khi[NM];
      static_for<PD>([&](auto I) {
        constexpr int m = I;
        constexpr int off = (m / 2) * 4 * ROW_BYTES + (m % 2) * 64;
        lds_read_b128<off>(klo[m], kaddr);
        lds_read_b128<off + 16>(khi[m], kaddr);
      });
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[kb][i] = 0.f;
      static_for<NM>([&](auto I) {
        constexpr int m = I;
        constexpr int younger = 2 * ((m + PD <= NM ? PD : NM - m) - 1);
        lds_wait2<younger>(klo[m], khi[m]);
        i32x8 kf = __builtin_shufflevector(klo[m], khi[m], 0, 1, 2, 3, 4, 5, 6, 7);
        sacc[m / 2] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf, qf[m % 2], sacc[m / 2], 0, 0, 0, 0, 0, 0);
        if constexpr (m + PD < NM) {
          constexpr int n = m + PD;
          constexpr int off = (n / 2) * 4 * ROW_BYTES + (n % 2) * 64;
          lds_read_b128<off>(klo[n], kaddr);
          lds_read_b128<off + 16>(khi[n], kaddr);
        }
      });
    }

    const int valid = (t < nt1) ? p.Sk - t * kKeysPerTile : p.Sk2 - (t - nt1) * kKeysPerTile;
    if (valid < kKeysPerTile) {
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          int key = 32 * kb + 8 * (i >> 2) + 4 * hh + (i & 3);
          if (key >= valid) sacc[kb][i] = -INFINITY;
        }
    }

    // ---- online softmax ---------------------------------------------------------------
    float mx = sacc[0][0];
#pragma unroll
    for (int i = 1; i < 16; i++) mx = fmaxf(mx, sacc[0][i]);
#pragma unroll
    for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[1][i]);
    mx = max_halves(mx);
    const float m_new = fmaxf(m_used, mx);
    const bool grow = (m_new - m_used) * c > kLazyRescaleLog2;
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float alpha = fast_exp2((m_used - m_new) * c);
      m_used = m_new;
      l_part *= alpha;
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
    }
    const float mc = m_used * c - kPShift;
    i32x8 pf;  // P^T: byte 16kb + i
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {
#pragma unroll
      for (int i = 0; i < 16; i += 4) {
        float p0 = fast_exp2(__builtin_fmaf(sacc[kb][i], c, -mc));
        float p1 = fast_exp2(__builtin_fmaf(sacc[kb][i + 1], c, -mc));
        float p2 = fast_exp2(__builtin_fmaf(sacc[kb][i + 2], c, -mc));
        float p3 = fast_exp2(__builtin_fmaf(sacc[kb][i + 3], c, -mc));
        l_part += (p0 + p1) + (p2 + p3);
        int w;  // both halves are written below: no need to clear the register first
        asm volatile("" : "=v"(w));
        w = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, w, true);
        pf[4 * kb + (i >> 2)] = w;
      }
    }

    // ---- O^T += V^T P^T ------------------------------------------------------------------
    // Four MFMAs (d blocks); each takes its V^T operand as four transposing 8-byte reads.
    {
      constexpr int PD = kPrefetch;
      constexpr int NM = 4;
      const unsigned vaddr = (unsigned)(uintptr_t)vtile;
      i32x2 vr[NM][4];
      static_for<PD>([&](auto I) {
        constexpr int m = I;
        static_for<4>([&](auto R) {
          constexpr int r = R;
          lds_read_tr8_b64<r * 2 * ROW_BYTES + m * 32>(vr[m][r], vaddr);
        });
      });
      static_for<NM>([&](auto I) {
        constexpr int m = I;
        constexpr int younger = 4 * ((m + PD <= NM ? PD : NM - m) - 1);
        lds_wait4<younger>(vr[m][0], vr[m][1], vr[m][2], vr[m][3]);
        i32x8 vf;
#pragma unroll
        for (int r = 0; r < 4; r++) {
          vf[2 * r] = vr[m][r][0];
          vf[2 * r + 1] = vr[m][r][1];
        }
        oacc[m] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf, oacc[m], 0, 0, 0, 0, 0, 0);
        if constexpr (m + PD < NM) {
          constexpr int n = m + PD;
          static_for<4>([&](auto R) {
            constexpr int r = R;
            lds_read_tr8_b64<r * 2 * ROW_BYTES + n * 32>(vr[n][r], vaddr);
          });
        }
      });
    }
  }

  // ---- epilogue -----------------------------------------------------------------------------
  const float l_tot = sum_halves(l_part);
  const float inv = sv / l_tot;
  const float lse = (m_used * c - kPShift + fast_log2(l_tot)) * kLn2;
  if (qrow < p.Sq) {
    TO* optr;
    if (part_out != nullptr) optr = part_out + (wave * kRowsPerWave + l32) * D;
    else optr = (TO*)p.out + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_s;
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
      for (int a = 0; a < 4; a++) {
        typedef __attribute__((ext_vector_type(4))) TO vec4;
        f32x4 o = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv,
                   oacc[db][4 * a + 3] * inv};
        vec4 ov = __builtin_convertvector(o, vec4);
        *(vec4*)(optr + 32 * db + 8 * a + 4 * hh) = ov;
      }
    if (hh == 0) {
      if (part_out != nullptr) part_lse[wave * kRowsPerWave + l32] = lse;
      else if (p.lse != nullptr) p.lse[b * p.ls_b + h * p.ls_h + qrow] = lse;
    }
  }
}

template <typename TO, int NW>
__global__ __launch_bounds__(64 * NW, NW == 8 ? 2 : 3) void attn_fwd_fp8_kernel(const AttnParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * BUF_BYTES];
  run_workgroup<TO, kRowsPerWave * NW, D>(p, [&](int tile, int it0, int it1, TO* part_out, float* part_lse) {
    attn_segment_fp8<TO, NW>(p, smem, tile, it0, it1, part_out, part_lse);
  });
}

// Workgroups of NW wavefronts resident at once (3 wavefronts per SIMD by registers; 2 for NW = 8).
static int resident_workgroups(int NW, int planned_cus) { return resident_cus(planned_cus) * (NW == 4 ? 3 : 1); }

template <typename TO, int NW>
static hipError_t launch_one(const AttnParams& p, hipStream_t stream) {
  AttnParams q = p;
  constexpr int rows = kRowsPerWave * NW;
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  bind_workspace(q, p, plan_split(q, rows, resident_workgroups(NW, p.cu_count), D, 2, 1), rows, D, 2);
  launch_counter_reset(q, stream);
  dim3 grid(split_grid(q));
  hipLaunchKernelGGL((attn_fwd_fp8_kernel<TO, NW>), grid, dim3(64 * NW), 0, stream, q);
  if (q.split_units) {
    const int nt = (q.Sk + kKeysPerTile - 1) / kKeysPerTile + (q.Sk2 + kKeysPerTile - 1) / kKeysPerTile;
    const dim3 cgrid((unsigned)((rows * (D / 8) + 255) / 256), (unsigned)(q.total_tiles - q.split_full));
    hipLaunchKernelGGL((attn_combine_kernel<TO, D>), cgrid, dim3(256), 0, stream, q, rows, nt, split_counters(q));
  }
  return hipGetLastError();
}

template <int NW>
static size_t workspace_one(const AttnParams& p, AttnParams* plan) {
  AttnParams q = p;
  constexpr int rows = kRowsPerWave * NW;
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  const size_t need = plan_split(q, rows, resident_workgroups(NW, p.cu_count), D, 2, 1);
  if (plan != nullptr) *plan = q;
  return need;
}

}  // namespace fp8path

// rows_per_block: 128 (4 wavefronts), 256 (8) or 384 (12 wavefronts sharing each K/V tile).
hipError_t launch_attn_fwd_fp8(const AttnParams& p, int out_is_fp16, int rows_per_block, hipStream_t stream) {
  using namespace fp8path;
  if (rows_per_block == 384) return out_is_fp16 ? launch_one<_Float16, 12>(p, stream) : launch_one<__bf16, 12>(p, stream);
  if (rows_per_block == 256) return out_is_fp16 ? launch_one<_Float16, 8>(p, stream) : launch_one<__bf16, 8>(p, stream);
  return out_is_fp16 ? launch_one<_Float16, 4>(p, stream) : launch_one<__bf16, 4>(p, stream);
}

size_t attn_fwd_fp8_workspace(const AttnParams& p, int rows_per_block, AttnParams* plan) {
  using namespace fp8path;
  if (rows_per_block == 384) return workspace_one<12>(p, plan);
  if (rows_per_block == 256) return workspace_one<8>(p, plan);
  return workspace_one<4>(p, plan);
}

}  // namespace xdit
