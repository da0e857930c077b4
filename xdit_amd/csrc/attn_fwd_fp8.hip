// Non-causal attention forward for fp8 (OCP e4m3fn) Q/K/V with per-(batch, head) fp32 descales,
// head_dim 128 or 64, bf16 or fp16 output, fp32 log-sum-exp, on gfx950.
//
// Same structure as the 16-bit kernel (workgroup = 4, 8 or 12 wavefronts x 32 query rows, 64-key
// K/V tiles double buffered in LDS by direct global->LDS loads, hand-issued LDS fragment reads,
// transposed products so that each lane owns one query), with v_mfma_f32_32x32x64_f8f6f4 for both products:
//   S^T = K Q^T    A = K rows, B = Q^T (registers); contraction over head_dim, 64 per instruction
//                  (two steps at head_dim 128, one at 64).
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
constexpr float kPShift = 6.0f;           // P is scaled by 2^6 ...
constexpr float kLazyRescaleLog2 = 2.0f;  // ... and the row max may lag by 2^2: P <= 2^8 < 448

// LDS tile geometry: rows of D bytes, 1024 / D rows per 1 KiB piece (what one wavefront
// instruction of the direct global->LDS load writes), NG pieces per 64-key tile; row r lives in
// piece r % NG at slot r / NG.  Piece pitches pad by 16 B (K: 16-byte reads of consecutive rows)
// and 32 B (V: 32-byte row segments) to spread the banks.
template <int D> struct Geom {
  static_assert(D == 128 || D == 64, "head_dim of the fp8 kernels");
  static constexpr int ROW_BYTES = D;
  static constexpr int NG = kKeysPerTile * D / 1024;   // 8 or 4
  static constexpr int K_PITCH = 1024 + 16;
  static constexpr int V_PITCH = 1024 + 32;
  static constexpr int K_BYTES = NG * K_PITCH;
  static constexpr int V_BYTES = NG * V_PITCH;
  static constexpr int BUF_BYTES = K_BYTES + V_BYTES;
  static constexpr int KS = D / 64;   // contraction steps of S^T
  static constexpr int DB = D / 32;   // 32-row blocks of O^T
};
// LDS fragment reads are issued this many MFMAs ahead of the MFMA that consumes them.
constexpr int kPrefetch = 2;

// Output staging block of a wavefront in the epilogue: 32 rows of 64 16-bit columns, rows 8 bytes
// apart from a multiple of 128 so that the 8-byte writes of the 32 lanes of a half hit 32 banks.
constexpr int kStagePitch = 64 * 2 + 8;
constexpr int kStageBytes = kRowsPerWave * kStagePitch + kRowsPerWave * 4;  // + one fp32 per row (ring step)
// LDS of a workgroup: the first K/V buffer, then a region that holds the second K/V buffer during
// the KV loop and the output staging blocks of the wavefronts in the epilogue.
template <int D, int NW>
constexpr int lds_bytes() { return Geom<D>::BUF_BYTES + (Geom<D>::BUF_BYTES > NW * kStageBytes ? Geom<D>::BUF_BYTES : NW * kStageBytes); }

// The work of one workgroup: its segments (WorkgroupWalk), one after the other; a segment is the
// query tile `tile` and KV tiles [it0, it1), written to the output tensors (slot < 0) or as one
// part of a shared query tile to its workspace slot.  As in the 16-bit kernel the kernel
// arguments are read in place (and afresh after every KV loop, so that the loop keeps the
// registers), the Q fragments and the first K/V tile of a workgroup's next segment are requested
// ahead of the epilogue of the current one, and the rows leave through an LDS transpose as
// whole 128-byte lines.
// FUSED: the ring step; the block (rounded to TO, what a block_out tensor would have held) is
// folded into the fp32 accumulator with the arithmetic of the merge kernel, so that the result
// equals forward + merge bit for bit; the parts of shared tiles go through the workspace as in a plain
// forward and are folded, then folded into the accumulator, by the fold duties.
template <typename TO, int D, int NW, bool FUSED>
__device__ __forceinline__ void attn_workgroup_fp8(unsigned char* smem) {
  typedef unsigned char u8;
  typedef Geom<D> G;
  constexpr int ROW_BYTES = G::ROW_BYTES, NG = G::NG, K_PITCH = G::K_PITCH, V_PITCH = G::V_PITCH, K_BYTES = G::K_BYTES,
                BUF_BYTES = G::BUF_BYTES, KS = G::KS, DB = G::DB;
  ParamsPtr pp = (ParamsPtr)__builtin_amdgcn_kernarg_segment_ptr();
  constexpr int kWaves = NW;
  constexpr int kRowsPerBlock = kRowsPerWave * kWaves;

  const int nt1 = (pp->Sk + kKeysPerTile - 1) / kKeysPerTile;
  const int nt = nt1 + (pp->Sk2 + kKeysPerTile - 1) / kKeysPerTile;
  __shared__ unsigned ticket;
  __shared__ unsigned fold_post;  // fold duties: the slices this workgroup folds, posted by thread 0
  WorkgroupWalk walk;
  Segment seg;
  {
    const WalkGeom g = walk_geom(pp);
    if (!walk.start(g, nt, (int)blockIdx.x) || !walk.next(g, nt, seg)) return;
  }
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int lane = lane_now();   // for the set-up below; later code asks again
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  // ---- tile loads ------------------------------------------------------------------------
  // Loader wavefronts: the first LW wavefronts each load PAIRS (K piece g, V piece g) pairs,
  // g = wave + LW * i, with one row index per lane for both pieces of a pair.
  constexpr int LW = kWaves < NG ? kWaves : NG;
  constexpr int PAIRS = NG / LW;
  constexpr int LANES_PER_ROW = ROW_BYTES / 16;
  int ld_row0 = NG * (lane / LANES_PER_ROW) + wave;    // row of this lane in pair 0
  unsigned ld_colb = (lane % LANES_PER_ROW) * 16;
  asm volatile("" : "+v"(ld_row0), "+v"(ld_colb));
  const unsigned lds_base = (unsigned)(uintptr_t)(XDIT_LDS u8*)smem;
  const unsigned ld_kdst = lds_base + wave * K_PITCH;  // LDS address of K piece `wave`, buffer 0
  const unsigned ld_vdst = lds_base + K_BYTES + wave * V_PITCH;

  // Where the K/V rows of the current (batch, head) lie, set per segment (row strides in bytes).
  const u8* kv_k1;
  const u8* kv_v1;
  const u8* kv_k2;
  const u8* kv_v2;
  unsigned kss1, vss1, kss2, vss2;
  int keys1, keys2;
  auto issue_tile = [&](int t, int buf) {
    if (kWaves == LW || wave < LW) {
      const bool second = t >= nt1;
      const unsigned row0 = (unsigned)(second ? t - nt1 : t) * kKeysPerTile;
      const unsigned kss = second ? kss2 : kss1, vss = second ? vss2 : vss1;
      const u8* kp = (second ? kv_k2 : kv_k1) + (uint64_t)row0 * kss;
      const u8* vp = (second ? kv_v2 : kv_v1) + (uint64_t)row0 * vss;
      const int left = (second ? keys2 : keys1) - (int)row0;
      const int last = (left < kKeysPerTile ? left : kKeysPerTile) - 1;
      const unsigned bo = buf * BUF_BYTES;
#pragma unroll
      for (int i = 0; i < PAIRS; i++) {
        int r = ld_row0 + LW * i;
        r = r < last ? r : last;  // rows past the end of the segment re-read its last row
        load_lds_16(kp, __umul24((unsigned)r, kss) + ld_colb, ld_kdst + bo + i * LW * K_PITCH);
        load_lds_16(vp, __umul24((unsigned)r, vss) + ld_colb, ld_vdst + bo + i * LW * V_PITCH);
      }
    }
  };

  // ---- LDS read bases ------------------------------------------------------------------------
  // K fragment for key block kb, step ks: row 32kb + l32, bytes 64ks + 32hh .. +31.
  unsigned kbase_off = lds_base + (l32 % NG) * K_PITCH + (l32 / NG) * ROW_BYTES + hh * 32;
  constexpr int K_KB_STEP = (32 / NG) * ROW_BYTES;   // +32 rows = +32/NG slots
  // V^T fragment, read r (0..3), d block db: as a SOURCE lane of ds_read_b64_tr_b8, lane
  // (group g = lane/16, s = lane%16) supplies 8 bytes of key row 16r + 8(s/8) + 4hh + (s/2)%4
  // at d = 32db + 16(g%2) + 8(s%2); lane (g, i) receives d = 32db + 16(g%2) + i for the 8 keys
  // 16r + 8(j/4) + 4hh + j%4, j = 0..7.
  const int s16 = lane & 15;
  const int vrow0 = 8 * (s16 >> 3) + 4 * hh + ((s16 >> 1) & 3);   // key row of read 0; read r is 16 r further
  unsigned vbase_off = lds_base + K_BYTES + (vrow0 % NG) * V_PITCH + (vrow0 / NG) * ROW_BYTES +
                       16 * ((lane >> 4) & 1) + 8 * (s16 & 1);
  constexpr int V_R_STEP = (16 / NG) * ROW_BYTES;    // +16 rows
  asm volatile("" : "+v"(kbase_off), "+v"(vbase_off));  // one register each through the loop

  // ---- per segment: coordinates, Q fragments (2 contraction steps x 32 bytes), scales, first tile
  int b, h, qt;
  float c, sv;
  i32x8 qf[KS];
  auto open_segment = [&](const Segment& sg) {
    const int lane = lane_now(), l32 = lane & 31, hh = lane >> 5;
    const int nq_tiles = pp->nq_tiles, H = pp->H;
    const int bh = sg.tile / nq_tiles;
    qt = sg.tile - bh * nq_tiles;
    b = bh / H;
    h = bh - b * H;
    kv_k1 = (const u8*)pp->k + b * pp->ks_b + h * pp->ks_h;
    kv_v1 = (const u8*)pp->v + b * pp->vs_b + h * pp->vs_h;
    kss1 = (unsigned)pp->ks_s; vss1 = (unsigned)pp->vs_s;
    keys1 = pp->Sk; keys2 = pp->Sk2;
    if (keys2 > 0) {
      kv_k2 = (const u8*)pp->k2 + b * pp->k2s_b + h * pp->k2s_h;
      kv_v2 = (const u8*)pp->v2 + b * pp->v2s_b + h * pp->v2s_h;
      kss2 = (unsigned)pp->k2s_s; vss2 = (unsigned)pp->v2s_s;
    } else {
      kv_k2 = kv_k1; kv_v2 = kv_v1; kss2 = kss1; vss2 = vss1;
    }
    float sq = 1.f, sk = 1.f;
    sv = 1.f;
    const int64_t ds = b * pp->ds_b + h * pp->ds_h;
    if (pp->q_descale) sq = pp->q_descale[ds];
    if (pp->k_descale) sk = pp->k_descale[ds];
    if (pp->v_descale) sv = pp->v_descale[ds];
    c = pp->scale * sq * sk * kLog2e;
    const int Sq = pp->Sq;
    const int qrow = qt * kRowsPerBlock + wave * kRowsPerWave + l32;
    const int qrow_c = qrow < Sq ? qrow : Sq - 1;
    const u8* qptr = (const u8*)pp->q + b * pp->qs_b + h * pp->qs_h + (int64_t)qrow_c * pp->qs_s + hh * 32;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      i32x4 lo = *(const i32x4*)(qptr + ks * 64);
      i32x4 hi = *(const i32x4*)(qptr + ks * 64 + 16);
      qf[ks] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    issue_tile(sg.it0, 0);
  };
  open_segment(seg);
  for (;;) {  // segments of this workgroup
    const int cb = b, ch = h, cqt = qt;
    const float cc = c, csv = sv;
    TO* part_out = nullptr;
    float* part_lse = nullptr;
    if (seg.slot >= 0) {
      part_out = (TO*)pp->ws_out + seg.slot * kRowsPerBlock * D;
      part_lse = pp->ws_lse + seg.slot * kRowsPerBlock;
    }
    const int keys_1 = keys1, keys_2 = keys2;
    float m_used = -INFINITY;
    float l_part = 0.f;
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(qf[ks]));

    for (int t = seg.it0; t < seg.it1; t++) {
      const int buf = (t - seg.it0) & 1;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (t + 1 < seg.it1) issue_tile(t + 1, buf ^ 1);

      const unsigned kaddr = kbase_off + buf * BUF_BYTES;
      const unsigned vaddr = vbase_off + buf * BUF_BYTES;

      // ---- S^T = K Q^T ---------------------------------------------------------------------
      // 2 KS MFMAs; MFMA m = 2 ks + kb (consecutive ones share their Q fragment) takes the 32 bytes
      // of its K row as two 16-byte reads.
      f32x16 sacc[2];
      {
        constexpr int PD = kPrefetch;  // MFMAs whose two reads are in flight
        constexpr int NM = 2 * KS;
        i32x4 klo[NM], khi[NM];
        static_for<PD>([&](auto I) {
          constexpr int m = I;
          constexpr int off = (m % 2) * K_KB_STEP + (m / 2) * 64;
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
          sacc[m % 2] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf, qf[m / 2], sacc[m % 2], 0, 0, 0, 0, 0, 0);
          if constexpr (m + PD < NM) {
            constexpr int n = m + PD;
            constexpr int off = (n % 2) * K_KB_STEP + (n / 2) * 64;
            lds_read_b128<off>(klo[n], kaddr);
            lds_read_b128<off + 16>(khi[n], kaddr);
          }
        });
      }

      const int valid = (t < nt1) ? keys_1 - t * kKeysPerTile : keys_2 - (t - nt1) * kKeysPerTile;
      if (valid < kKeysPerTile) {
        const int hh = lane_now() >> 5;
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
      const bool grow = (m_new - m_used) * cc > kLazyRescaleLog2;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float alpha = fast_exp2((m_used - m_new) * cc);
        m_used = m_new;
        l_part *= alpha;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
      }
      const float mc = m_used * cc - kPShift;
      i32x8 pf;  // P^T: byte 16kb + i
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
          float p0 = fast_exp2(__builtin_fmaf(sacc[kb][i], cc, -mc));
          float p1 = fast_exp2(__builtin_fmaf(sacc[kb][i + 1], cc, -mc));
          float p2 = fast_exp2(__builtin_fmaf(sacc[kb][i + 2], cc, -mc));
          float p3 = fast_exp2(__builtin_fmaf(sacc[kb][i + 3], cc, -mc));
          l_part += (p0 + p1) + (p2 + p3);
          int w;  // both halves are written below: no need to clear the register first
          asm volatile("" : "=v"(w));
          w = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, w, false);
          w = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, w, true);
          pf[4 * kb + (i >> 2)] = w;
        }
      }

      // ---- O^T += V^T P^T ------------------------------------------------------------------
      // One MFMA per d block; each takes its V^T operand as four transposing 8-byte reads.
      {
        constexpr int PD = kPrefetch;
        constexpr int NM = DB;
        i32x2 vr[NM][4];
        static_for<PD>([&](auto I) {
          constexpr int m = I;
          static_for<4>([&](auto R) {
            constexpr int r = R;
            lds_read_tr8_b64<r * V_R_STEP + m * 32>(vr[m][r], vaddr);
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
              lds_read_tr8_b64<r * V_R_STEP + n * 32>(vr[n][r], vaddr);
            });
          }
        });
      }
    }
    asm volatile("" : "+s"(pp));  // from here on the kernel arguments are read afresh

    // ---- what comes next for this workgroup --------------------------------------------------
    Segment next_seg;
    bool more;
    {
      const WalkGeom g = walk_geom(pp);
      unsigned* const range_counter = pp->split_counter;
      if (walk.wants_claim(range_counter != nullptr)) {
        __syncthreads();  // everyone has read the ticket of the previous claim
        if (wave == 0 && lane_now() == 0) ticket = atomicAdd(range_counter, 1u);
        __syncthreads();
        walk.claimed(g, (unsigned)__builtin_amdgcn_readfirstlane((int)ticket));
      }
      more = walk.next(g, nt, next_seg);
    }
    __syncthreads();  // every wavefront is done with the K/V fragments of the last tile
    if (more) open_segment(next_seg);  // Q fragments and first K/V tile (buffer 0) of the next segment

    // ---- epilogue: rows through an LDS transpose, 64 columns at a time --------------------------
    const int lane = lane_now(), l32 = lane & 31, hh = lane >> 5;
    const int cqrow = cqt * kRowsPerBlock + wave * kRowsPerWave + l32;
    const float l_tot = sum_halves(l_part);
    const float inv = csv / l_tot;
    const float lse = (m_used * cc - kPShift + fast_log2(l_tot)) * kLn2;
    typedef __attribute__((ext_vector_type(4))) TO vec4;
    typedef __attribute__((ext_vector_type(8))) TO vec8;
    XDIT_LDS unsigned char* stage = (XDIT_LDS unsigned char*)smem + BUF_BYTES + wave * kStageBytes;
    const int row0 = cqt * kRowsPerBlock + wave * kRowsPerWave;
    if (!FUSED || part_out != nullptr) {
      TO* obase;
      int64_t ostride;
      int rows_live = kRowsPerWave;
      if (part_out != nullptr) {
        obase = part_out + (int64_t)(wave * kRowsPerWave) * D;
        ostride = D;
      } else {
        obase = (TO*)pp->out + cb * pp->os_b + ch * pp->os_h + (int64_t)row0 * pp->os_s;
        ostride = pp->os_s;
        rows_live = pp->Sq - row0;  // may be <= 0 or above 32
      }
      const int rd_row = lane >> 3;          // + 8r
      const int rd_col = (lane & 7) * 8;     // element column within the 64-column pass
#pragma unroll
      for (int half = 0; half < D / 64; half++) {
#pragma unroll
        for (int dbl = 0; dbl < 2; dbl++) {
          const int db = 2 * half + dbl;
#pragma unroll
          for (int a = 0; a < 4; a++) {
            f32x4 o = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv,
                       oacc[db][4 * a + 3] * inv};
            *(XDIT_LDS vec4*)(stage + l32 * kStagePitch + (32 * dbl + 8 * a + 4 * hh) * 2) = __builtin_convertvector(o, vec4);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int row = rd_row + 8 * r;
          const vec8 x = *(const XDIT_LDS vec8*)(stage + row * kStagePitch + rd_col * 2);
          if (row < rows_live) {
            if (FUSED && part_out != nullptr) store16_device(obase + row * ostride + 64 * half + rd_col, __builtin_bit_cast(i32x4, x));  // read by another workgroup of this launch
            else __builtin_nontemporal_store(x, (vec8*)(obase + row * ostride + 64 * half + rd_col));
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      if (hh == 0 && cqrow < pp->Sq) {
        if (part_out != nullptr) { if (FUSED) store_float_device(part_lse + wave * kRowsPerWave + l32, lse); else part_lse[wave * kRowsPerWave + l32] = lse; }
        else if (pp->lse != nullptr) pp->lse[cb * pp->ls_b + ch * pp->ls_h + cqrow] = lse;
      }
    } else {
      // the block goes through the same LDS transpose, so that the accumulator is read and written
      // in whole rows; the weight of each row's fold travels with it
      XDIT_LDS float* wrow = (XDIT_LDS float*)(stage + kRowsPerWave * kStagePitch);
      const bool first = pp->acc_first != 0;
      float* alp = pp->acc_lse + cb * pp->al_b + ch * pp->al_h + (int64_t)cqrow * pp->al_s;
      float w = 0.f, new_lse = lse;
      if (!first && cqrow < pp->Sq) {
        const float la = *alp;
        w = sigmoid(lse - la);
        new_lse = la - log_sigmoid(la - lse);
      }
      if (hh == 0) wrow[l32] = w;
      float* abase = pp->acc_out + cb * pp->ao_b + ch * pp->ao_h + (int64_t)row0 * pp->ao_s;
      TO* obase = pp->out != nullptr ? (TO*)pp->out + cb * pp->os_b + ch * pp->os_h + (int64_t)row0 * pp->os_s : nullptr;
      const int rows_live = pp->Sq - row0;
      const int rd_row = lane >> 3;
      const int rd_col = (lane & 7) * 8;
#pragma unroll
      for (int half = 0; half < D / 64; half++) {
#pragma unroll
        for (int dbl = 0; dbl < 2; dbl++) {
          const int db = 2 * half + dbl;
#pragma unroll
          for (int a = 0; a < 4; a++) {
            f32x4 o = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv,
                       oacc[db][4 * a + 3] * inv};
            *(XDIT_LDS vec4*)(stage + l32 * kStagePitch + (32 * dbl + 8 * a + 4 * hh) * 2) = __builtin_convertvector(o, vec4);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int row = rd_row + 8 * r;
          const int col = 64 * half + rd_col;
          const vec8 x = *(const XDIT_LDS vec8*)(stage + row * kStagePitch + rd_col * 2);
          const float wr = wrow[row];
          if (row < rows_live) {
            float* aptr = abase + row * pp->ao_s + col;
            f32x4 m0, m1;
#pragma unroll
            for (int e = 0; e < 4; e++) { m0[e] = (float)x[e]; m1[e] = (float)x[4 + e]; }
            if (!first) {
              const f32x4 a0 = *(const f32x4*)aptr, a1 = *(const f32x4*)(aptr + 4);
#pragma unroll
              for (int e = 0; e < 4; e++) { m0[e] = fold_value(a0[e], m0[e], wr); m1[e] = fold_value(a1[e], m1[e], wr); }
            }
            if (pp->acc_store) { *(f32x4*)aptr = m0; *(f32x4*)(aptr + 4) = m1; }
            if (obase != nullptr) {
              vec8 y;
#pragma unroll
              for (int e = 0; e < 4; e++) { y[e] = (TO)m0[e]; y[4 + e] = (TO)m1[e]; }
              *(vec8*)(obase + row * pp->os_s + col) = y;
            }
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      if (hh == 0 && cqrow < pp->Sq) {
        *alp = new_lse;
        if (pp->lse != nullptr) pp->lse[cb * pp->ls_b + ch * pp->ls_h + cqrow] = new_lse;
      }
    }
    if constexpr (FUSED && NW != 12) if (seg.slot >= 0 && pp->split_fold != 0) {
      // this part of a shared tile is written: its arrival, with its fold duty unless that waits for the workgroup's end
      const WalkGeom g = walk_geom(pp);
      const int r = seg.tile - g.split_full;
      const int j = (int)(seg.slot - (int64_t)r * g.split_pmax);
      const int n = shared_tile_parts(g, nt, r);
      const bool now = g.split_order == 0;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's rows of the partial result have been written through
      fold_arrival<TO, D, kRowsPerBlock, FUSED>(pp, nt, r, j, n, now, &fold_post);
    }
    if (!more) break;
    seg = next_seg;
  }
  if constexpr (FUSED && NW != 12) if (pp->split_fold != 0) {
    if (pp->split_order != 0) fold_duties_at_end<TO, D, kRowsPerBlock, FUSED>(pp, nt, &fold_post);
    if (walk.claimer && pp->split_counter != nullptr && pp->split_dyn == 0) claimer_done(pp);
  }
}

template <typename TO, int D, int NW, bool FUSED>
__global__ __launch_bounds__(64 * NW, NW == 8 ? 2 : 3) void attn_fwd_fp8_kernel(const AttnParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // [K tile | V tile] [K tile | V tile, or output staging]
  attn_workgroup_fp8<TO, D, NW, FUSED>(smem);
}

// Workgroups of NW wavefronts resident at once (3 wavefronts per SIMD by registers; 2 for NW = 8).
static int resident_workgroups(int NW, int planned_cus) { return resident_cus(planned_cus) * (NW == 4 ? 3 : 1); }

template <typename TO, int D, int NW, bool FUSED>
static hipError_t launch_one(const AttnParams& p, hipStream_t stream) {
  AttnParams q = p;
  constexpr int rows = kRowsPerWave * NW;
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  // the ring step takes a balanced plan only when the attention kernel folds the parts itself (the fold goes on into the accumulator)
  bind_workspace(q, p, plan_split(q, rows, resident_workgroups(NW, p.cu_count), D, 2, 1, false, FUSED), rows, D, 2);
  static std::atomic<bool> lds_ready[kMaxDevices];
  constexpr int lds = lds_bytes<D, NW>();
  const int slot = current_device_slot();
  if (lds > 65536 && !lds_ready[slot].load(std::memory_order_relaxed)) {  // > 64 KiB of dynamic LDS must be enabled once per kernel and device
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_fp8_kernel<TO, D, NW, FUSED>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    lds_ready[slot].store(true, std::memory_order_relaxed);
  }
  dim3 grid(split_grid(q));
  hipLaunchKernelGGL((attn_fwd_fp8_kernel<TO, D, NW, FUSED>), grid, dim3(64 * NW), lds, stream, q);
  if constexpr (!FUSED) {
    if (q.split_units && !q.split_fold) {  // tiles of many parts: folded by a launch of its own
      const int nt = (q.Sk + kKeysPerTile - 1) / kKeysPerTile + (q.Sk2 + kKeysPerTile - 1) / kKeysPerTile;
      const dim3 cgrid((unsigned)((rows * (D / 8) + 255) / 256), (unsigned)(q.total_tiles - q.split_full));
      hipLaunchKernelGGL((attn_combine_kernel<TO, D>), cgrid, dim3(256), 0, stream, q, rows, nt, split_counters(q));
    }
  }
  return hipGetLastError();
}

template <int D, int NW>
static size_t workspace_one(const AttnParams& p, AttnParams* plan, bool fold_only) {
  AttnParams q = p;
  constexpr int rows = kRowsPerWave * NW;
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  const size_t need = plan_split(q, rows, resident_workgroups(NW, p.cu_count), D, 2, 1, false, fold_only);
  if (plan != nullptr) *plan = q;
  return need;
}

}  // namespace fp8path

// rows_per_block: 128 (4 wavefronts), 256 (8) or 384 (12 wavefronts sharing each K/V tile).
template <int D, bool FUSED>
static hipError_t launch_fp8(const AttnParams& p, int out_is_fp16, int rows_per_block, hipStream_t stream) {
  using namespace fp8path;
  if (rows_per_block == 384) return out_is_fp16 ? launch_one<_Float16, D, 12, FUSED>(p, stream) : launch_one<__bf16, D, 12, FUSED>(p, stream);
  if (rows_per_block == 256) return out_is_fp16 ? launch_one<_Float16, D, 8, FUSED>(p, stream) : launch_one<__bf16, D, 8, FUSED>(p, stream);
  return out_is_fp16 ? launch_one<_Float16, D, 4, FUSED>(p, stream) : launch_one<__bf16, D, 4, FUSED>(p, stream);
}

// D: 128 or 64.  p.acc_out set: the ring step (fold into the fp32 accumulator in the epilogue).
hipError_t launch_attn_fwd_fp8(const AttnParams& p, int D, int out_is_fp16, int rows_per_block, hipStream_t stream) {
  if (D == 128) return p.acc_out != nullptr ? launch_fp8<128, true>(p, out_is_fp16, rows_per_block, stream) : launch_fp8<128, false>(p, out_is_fp16, rows_per_block, stream);
  if (D == 64) return p.acc_out != nullptr ? launch_fp8<64, true>(p, out_is_fp16, rows_per_block, stream) : launch_fp8<64, false>(p, out_is_fp16, rows_per_block, stream);
  return hipErrorInvalidValue;
}

size_t attn_fwd_fp8_workspace(const AttnParams& p, int D, int rows_per_block, AttnParams* plan, bool fold_only) {
  using namespace fp8path;
  if (D == 128) {
    if (rows_per_block == 384) return workspace_one<128, 12>(p, plan, fold_only);
    if (rows_per_block == 256) return workspace_one<128, 8>(p, plan, fold_only);
    return workspace_one<128, 4>(p, plan, fold_only);
  }
  if (rows_per_block == 384) return workspace_one<64, 12>(p, plan, fold_only);
  if (rows_per_block == 256) return workspace_one<64, 8>(p, plan, fold_only);
  return workspace_one<64, 4>(p, plan, fold_only);
}

}  // namespace xdit
