// Non-causal attention forward for 16-bit inputs (bf16 / fp16) on gfx950, built for head_dim 64 and 128
// (tensors of a smaller head_dim, a multiple of 8, run on the next one up: see PAD below).
//
// Work decomposition
//   workgroup = NW wavefronts (4, 8 or 12); a query tile is 32 NW rows of one (batch, head) and
//   wavefront w owns rows [32w, 32w+32) of it.  Keys/values stream through LDS in tiles of 64
//   keys, double buffered, filled by direct global->LDS loads (16 bytes per lane).  A workgroup
//   is persistent: it walks the segments (whole query tiles, shares of shared ones) that
//   WorkgroupWalk deals it.
//
// MFMA orientation (v_mfma_f32_32x32x16_{bf16,f16}; A is 32x16, B is 16x32, lane l holds row/col
// l%32 and the 8 contraction elements 8*(l/32)..+7; the 32x32 result puts column l%32 and rows
// 8*(i/4) + 4*(l/32) + i%4, i = 0..15, in lane l):
//   S^T = K Q^T    A = K tile rows (keys), B = Q^T (kept in registers for the whole kernel)
//   O^T = V^T P^T  A = V^T (read transposed from LDS with ds_read_b64_tr_b16), B = P^T
// Computing the transposed products makes every lane own ONE query (column l%32): the softmax
// row statistics are per-lane scalars (one exchange between the two wavefront halves per tile),
// and the S^T accumulator registers are, after conversion to 16 bit, exactly the B operand of
// the second product, so P never goes through LDS.
//
// LDS layout: see attn_tiles.h.  The workgroup has NW = 4, 8 or 12 wavefronts (128 / 256 / 384
// query rows): 8 or 12 wavefronts share every K/V tile, which cuts the L2->LDS traffic per FLOP
// to a half or a third, and are used when the problem still yields enough workgroups to fill
// the chip.
//
// LDS fragment reads are issued by hand (inline assembly, kPrefetch MFMAs ahead of their use,
// completion awaited with counted s_waitcnt): left to the compiler, every MFMA waits for a read
// issued just before it, and the read latency is paid sixteen times per product and tile.
#pragma once
#include "attn_split.h"
#include "launchers.h"

// Timestamp hooks of an instrumented build: a translation unit that defines XDIT_TRACE_POINT(part, k)
// before including this file records when a workgroup passes point k (0 entry of a segment,
// 1 first K/V tile landed, 2 end of the KV loop, 3 end of the epilogue); nothing otherwise.
#ifndef XDIT_TRACE_POINT
#define XDIT_TRACE_POINT(part, k)
#endif

namespace xdit {

constexpr int kRowsPerWave = 32;
// LDS fragment reads are issued this many MFMAs ahead of the MFMA that consumes them.
constexpr int kPrefetch = 4;

// Output staging block of a wavefront in the epilogue: 32 rows of 64 16-bit columns, rows 8 bytes
// apart from a multiple of 128 so that the 8-byte writes of the 32 lanes of a half hit 32 banks.
constexpr int kStagePitchBytes = 64 * 2 + 8;
constexpr int kStageBytesPerWave = kRowsPerWave * kStagePitchBytes + kRowsPerWave * 4;  // + one fp32 per row (ring step)

// LDS of a workgroup: the first K/V buffer, then a region that holds the second K/V buffer during
// the KV loop and the output staging blocks of the wavefronts in the epilogue.  The epilogue thus
// leaves the first buffer alone, and the first K/V tile of the workgroup's next segment is loaded
// into it while the rows of the current one are stored.
template <int D, int NW>
constexpr int lds_bytes_16() {
  return TileGeom<D>::BUF_BYTES + (TileGeom<D>::BUF_BYTES > NW * kStageBytesPerWave ? TileGeom<D>::BUF_BYTES : NW * kStageBytesPerWave);
}

// The work of one workgroup: its segments (WorkgroupWalk), one after the other.  A segment is the
// query tile `tile` and KV tiles [it0, it1), plus, under streamed sharing, further KV tiles of the
// same query tile drawn one at a time from the tile's counter.  With slot < 0 the normalised
// result goes to the output tensors; otherwise the segment is one PART of a query tile whose KV
// range is shared between workgroups, and its normalised partial output (in T) and log-sum-exp
// go to the workspace slot, [row][D] and [row], to be folded by attn_combine_kernel.
// Between two segments the Q fragments and the first K/V tile of the next one are requested
// before the rows of the current one are stored, so their latency hides behind the epilogue.
// PAD: the tensors' head_dim (p.d_actual, a multiple of 8) is smaller than D; the missing columns
// are zeros in the Q fragments and in LDS (cleared once, never written by the tile loads) and are
// not stored.  DC (a multiple of 16, d_actual <= DC <= D) is the head_dim the two products are
// computed over: LDS tiles keep the geometry of D, contraction steps (of 16) and output blocks
// (of 32) past DC are left out.
// The kernel's only argument is read in place, through a pointer to the kernel-argument segment
// that is made opaque to the compiler after every KV loop: what a segment's prologue and
// epilogue need is then loaded (scalar loads) when it is needed instead of being kept in
// registers across the loop, which leaves the loop the registers.
template <typename T, int D, int DC, int NW, bool PAD, bool FUSED>
__device__ __forceinline__ void attn_workgroup(unsigned char* smem) {
  ParamsPtr pp = (ParamsPtr)__builtin_amdgcn_kernarg_segment_ptr();
  constexpr int kWaves = NW;
  constexpr int kRowsPerBlock = kRowsPerWave * kWaves;
  typedef typename Mfma16<T>::vec8 vec8;
  typedef typename Mfma16<T>::vec2 vec2;
  typedef TileGeom<D> G;
  static_assert(DC % 16 == 0 && DC <= D && (PAD || DC == D), "computed head_dim");
  constexpr int KSTEPS = DC / 16;          // contraction steps of QK^T
  constexpr int DBLOCKS = (DC + 31) / 32;  // 32-row blocks of O^T
  constexpr int kStagePitch = kStagePitchBytes;   // LDS row pitch of the output staging block
  constexpr int kStageBytes = kStageBytesPerWave;

  const int nt1 = (pp->Sk + kKeysPerTile - 1) / kKeysPerTile;
  const int nt = nt1 + (pp->Sk2 + kKeysPerTile - 1) / kKeysPerTile;
  __shared__ unsigned ticket;   // range claims
  __shared__ unsigned fold_post;  // fold duties: the slices this workgroup folds, posted by thread 0
  __shared__ int drawn[2];      // streamed sharing: KV tile of the stream position after next, by parity
  WorkgroupWalk walk;
  Segment seg;
  {
    const WalkGeom g = walk_geom(pp);
    if (!walk.start(g, nt, (int)blockIdx.x) || !walk.next(g, nt, seg)) return;
  }

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int dact = PAD ? pp->d_actual : D;
  const int lane = lane_now();   // for the set-up below; later code asks again
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  // ---- direct global->LDS tile loads ------------------------------------------------------
  // A tile is 2*NG pieces of 1 KiB (K pieces 0..NG-1, then V pieces): piece g of K (or V) holds
  // rows g, g+NG, g+2NG, ...; wavefront w loads pieces w, w+NW, w+2NW, ...; within a piece
  // lane -> (slot = lane / lanes-per-row, 16-byte column = lane % lanes-per-row).  A load is
  // "uniform 64-bit tile base + per-lane 32-bit byte offset".
  constexpr int LANES_PER_ROW = G::ROW_BYTES / 16;
  // Loader wavefronts: the first LW wavefronts each load PAIRS (K piece g, V piece g) pairs,
  // g = wave + LW * i, with one row index per lane for both pieces of a pair.
  constexpr int LW = kWaves < 8 ? kWaves : 8;
  constexpr int PAIRS = G::NG / LW;
  static_assert(G::NG % LW == 0, "pieces must divide evenly over the loader wavefronts");
  int ld_row0 = G::NG * (lane / LANES_PER_ROW) + wave;   // row of this lane in pair 0
  unsigned ld_colb = (lane % LANES_PER_ROW) * 16;        // byte offset inside the row
  asm volatile("" : "+v"(ld_row0), "+v"(ld_colb));       // kept as two registers through the KV loop
  const bool ld_on = !PAD || ld_colb < (unsigned)dact * 2;  // lanes of columns the tensors do not have stay idle
  const unsigned lds_base = (unsigned)(uintptr_t)(XDIT_LDS unsigned char*)smem;
  const unsigned ld_kdst = lds_base + wave * G::K_PITCH;      // LDS address of K piece `wave`, buffer 0
  const unsigned ld_vdst = lds_base + G::K_BYTES + wave * G::V_PITCH;

  // Where the K/V rows of the current (batch, head) lie, set per segment: per KV segment the
  // pointers to its first rows, the row strides in bytes (below 2^24) and its number of keys.
  const T* kv_k1;
  const T* kv_v1;
  const T* kv_k2;
  const T* kv_v2;
  unsigned kss1, vss1, kss2, vss2;
  int keys1, keys2;
  // Loads KV tile t of the current (batch, head) into buffer `buf`.
  auto issue_tile = [&](int t, int buf) {
    if ((kWaves == LW || wave < LW) && ld_on) {
      const bool second = t >= nt1;
      const unsigned row0 = (unsigned)(second ? t - nt1 : t) * kKeysPerTile;   // first key of the tile within its segment
      const unsigned kss = second ? kss2 : kss1, vss = second ? vss2 : vss1;
      const T* kp = (const T*)((const unsigned char*)(second ? kv_k2 : kv_k1) + (uint64_t)row0 * kss);
      const T* vp = (const T*)((const unsigned char*)(second ? kv_v2 : kv_v1) + (uint64_t)row0 * vss);
      const int left = (second ? keys2 : keys1) - (int)row0;
      const int last = (left < kKeysPerTile ? left : kKeysPerTile) - 1;
      const unsigned bo = buf * G::BUF_BYTES;
#pragma unroll
      for (int i = 0; i < PAIRS; i++) {
        int r = ld_row0 + LW * i;
        r = r < last ? r : last;  // rows past the end of the segment re-read its last row
        load_lds_16(kp, __umul24((unsigned)r, kss) + ld_colb, ld_kdst + bo + i * LW * G::K_PITCH);
        load_lds_16(vp, __umul24((unsigned)r, vss) + ld_colb, ld_vdst + bo + i * LW * G::V_PITCH);
      }
    }
  };

  // ---- LDS read addresses: one per-lane base each for K and V, the rest are immediates ------
  // K fragment (A operand of S^T) for key block kb, step ks: row 32kb + l32, bytes 32ks + 16hh.
  //   row -> piece (row % NG), slot (row / NG)
  unsigned kbase_off = lds_base + (l32 % G::NG) * G::K_PITCH + (l32 / G::NG) * G::ROW_BYTES + hh * 16;
  asm volatile("" : "+v"(kbase_off));  // one register, not its summands, lives through the loop
  constexpr int K_KB_STEP = (32 / G::NG) * G::ROW_BYTES;  // +32 rows = +32/NG slots
  // V^T fragment (A operand of O^T) for d block db, key step j (16 keys), half rd (keys +0 / +8):
  // as a SOURCE lane of the transposed read, lane (group g = lane/16, s = lane%16) supplies the
  // 8 bytes at key row 16j + 8rd + 4hh + s/4, elements d = 32db + 16(g%2) + 4(s%4) .. +3; the
  // read returns to lane (g, i) the four keys of that row group at d = 32db + 16(g%2) + i.
  const int vsrc_row = 4 * hh + ((lane & 15) >> 2);  // row within the 16-key step, rd = 0
  unsigned vbase_off = lds_base + G::K_BYTES + (vsrc_row % G::NG) * G::V_PITCH + (vsrc_row / G::NG) * G::ROW_BYTES +
                       (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  asm volatile("" : "+v"(vbase_off));
  // +8 rows (rd) and +16 rows (j): both keep row % NG pattern simple because NG is 8 or 16.
  constexpr int V_RD_STEP = (G::NG == 16) ? 8 * G::V_PITCH : G::ROW_BYTES;  // NG=8: +8 rows = +1 slot
  constexpr int V_J_STEP = (16 / G::NG) * G::ROW_BYTES;

  const float c = pp->scale * kLog2e;  // logits are kept in log2 units

  if (PAD) {  // zero the columns that no load writes (all of both buffers: simplest); once per workgroup
    typedef __attribute__((ext_vector_type(4))) int i32x4;
    const i32x4 zero = {0, 0, 0, 0};
    for (int i = (wave * 64 + lane) * 16; i < 2 * G::BUF_BYTES; i += 64 * kWaves * 16) *(XDIT_LDS i32x4*)((XDIT_LDS unsigned char*)smem + i) = zero;
    __syncthreads();
  }

  // ---- per segment: coordinates, Q fragments (B operand of S^T, lane = (query l32, contraction
  // half hh)) and the first K/V tile; issued here for the first segment and, for every later
  // one, ahead of the epilogue of its predecessor -------------------------------------------
  int b, h, qt;
  vec8 qf[KSTEPS];
  auto open_segment = [&](const Segment& sg) {
    const int lane = lane_now(), l32 = lane & 31, hh = lane >> 5;
    const int nq_tiles = pp->nq_tiles, H = pp->H;
    const int bh = sg.tile / nq_tiles;
    qt = sg.tile - bh * nq_tiles;
    b = bh / H;
    h = bh - b * H;
    kv_k1 = (const T*)pp->k + b * pp->ks_b + h * pp->ks_h;
    kv_v1 = (const T*)pp->v + b * pp->vs_b + h * pp->vs_h;
    kss1 = (unsigned)pp->ks_s * 2; vss1 = (unsigned)pp->vs_s * 2;
    keys1 = pp->Sk; keys2 = pp->Sk2;
    if (keys2 > 0) {
      kv_k2 = (const T*)pp->k2 + b * pp->k2s_b + h * pp->k2s_h;
      kv_v2 = (const T*)pp->v2 + b * pp->v2s_b + h * pp->v2s_h;
      kss2 = (unsigned)pp->k2s_s * 2; vss2 = (unsigned)pp->v2s_s * 2;
    } else {
      kv_k2 = kv_k1; kv_v2 = kv_v1; kss2 = kss1; vss2 = vss1;
    }
    const int Sq = pp->Sq;
    const int qrow = qt * kRowsPerBlock + wave * kRowsPerWave + l32;
    const int qrow_c = qrow < Sq ? qrow : Sq - 1;
    const T* qptr = (const T*)pp->q + b * pp->qs_b + h * pp->qs_h + (int64_t)qrow_c * pp->qs_s + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      if (!PAD || ks * 16 + hh * 8 < dact) {
        qf[ks] = *(const vec8*)(qptr + ks * 16);
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) qf[ks][e] = (T)0.f;
      }
    }
    issue_tile(sg.it0, 0);
  };
  XDIT_TRACE_POINT(seg.slot >= 0, 0);
  open_segment(seg);
  for (;;) {  // segments of this workgroup
    // Coordinates of the segment being computed (open_segment of the next one overwrites them).
    const int cb = b, ch = h, cqt = qt;
    T* part_out = nullptr;
    float* part_lse = nullptr;
    if (seg.slot >= 0) {
      part_out = (T*)pp->ws_out + seg.slot * kRowsPerBlock * D;
      part_lse = pp->ws_lse + seg.slot * kRowsPerBlock;
    }
    // Streamed sharing: stream position i holds KV tile it0 + i while i < n_own; later positions
    // are drawn from the tile's counter, two positions ahead of their use.
    const int n_own = seg.it1 - seg.it0;
    const bool streamed = seg.dyn >= 0;
    const int pool_len = nt - seg.pool0;
    unsigned* const draw_counter = streamed ? pp->split_counter + seg.dyn : nullptr;
    bool pool_open = streamed;  // thread 0: no ticket has come back past the end of the pool yet
    const int keys_1 = keys1, keys_2 = keys2;

    // ---- online softmax state: one query per lane (both halves of the wavefront agree) ------
    float m_used = -INFINITY;          // running (lazily updated) row maximum of the raw dot products
    float l_part = 0.f;                // this lane's share of the running row sum
    f32x16 oacc[DBLOCKS];
#pragma unroll
    for (int db = 0; db < DBLOCKS; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;

    // Make the compiler account for the Q fragment loads here, before the loop: the tile loads
    // are invisible to its outstanding-load bookkeeping, so any wait it placed for a Q fragment
    // inside the loop would also wait for the prefetch of the next tile.
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) asm volatile("" : "+v"(qf[ks]));

    int t = seg.it0;
    for (int i = 0;; i++) {
      const int buf = i & 1;
      // Tile t has landed (this thread's loads) and, after the barrier, everyone's; the barrier
      // also means every wavefront is done reading the other buffer, which the next tile now
      // overwrites.  A ticket drawn during the previous iteration has come back as well: thread
      // 0 posts the KV tile it stands for (position i + 1) before the barrier.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (i == 0) { XDIT_TRACE_POINT(seg.slot >= 0, 1); }
      int t_next;
      if (i + 1 < n_own) t_next = t + 1;
      else if (streamed) t_next = __builtin_amdgcn_readfirstlane(drawn[(i + 1) & 1]);  // posted during the previous iteration
      else t_next = -1;
      if (t_next >= 0) issue_tile(t_next, buf ^ 1);
      // Streamed sharing: thread 0 draws the ticket of position i + 2 now and posts the KV tile
      // it stands for at the end of this iteration, when the ticket has long come back.
      const bool drawing = streamed && i + 2 >= n_own && t_next >= 0;
      unsigned draw = 0xffffffffu;
      if (drawing && wave == 0 && pool_open && lane_now() == 0) draw = draw_ticket(draw_counter);

      const unsigned kaddr = kbase_off + buf * G::BUF_BYTES;
      const unsigned vaddr = vbase_off + buf * G::BUF_BYTES;

      // ---- S^T = K Q^T : 2 blocks of 32 keys x 32 queries ---------------------------------
      f32x16 sacc[2];
      {
        constexpr int PD = kPrefetch;   // K fragment reads in flight
        constexpr int NR = 2 * KSTEPS;  // reads (= MFMAs) of this product
        vec8 kf[NR];  // in MFMA order: contraction step i / 2 of key block i % 2, so that consecutive MFMAs share their Q fragment
        static_for<PD>([&](auto I) {
          constexpr int i_ = I;
          lds_read_b128<(i_ % 2) * K_KB_STEP + (i_ / 2) * 32>(kf[i_], kaddr);
        });
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int e = 0; e < 16; e++) sacc[kb][e] = 0.f;
        static_for<NR>([&](auto I) {
          constexpr int i_ = I;
          constexpr int younger = (i_ + PD <= NR ? PD : NR - i_) - 1;
          lds_wait<younger>(kf[i_]);
          sacc[i_ % 2] = Mfma16<T>::mma(kf[i_], qf[i_ / 2], sacc[i_ % 2]);
          if constexpr (i_ + PD >= NR && i_ + 1 < NR) __builtin_amdgcn_sched_barrier(0);  // issued before the next wait, not after the last one
          if constexpr (i_ + PD < NR) {
            constexpr int n = i_ + PD;
            lds_read_b128<(n % 2) * K_KB_STEP + (n / 2) * 32>(kf[n], kaddr);
          }
        });
      }
      // ---- mask keys past the end of the segment (only its last tile can be partial) -------
      const int valid = (t < nt1) ? keys_1 - t * kKeysPerTile : keys_2 - (t - nt1) * kKeysPerTile;
      if (valid < kKeysPerTile) {
        const int hh = lane_now() >> 5;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int e = 0; e < 16; e++) {
            int key = 32 * kb + 8 * (e >> 2) + 4 * hh + (e & 3);
            if (key >= valid) sacc[kb][e] = -INFINITY;
          }
      }

      // ---- online softmax ---------------------------------------------------------------
      float mx = sacc[0][0];
#pragma unroll
      for (int e = 1; e < 16; e++) mx = fmaxf(mx, sacc[0][e]);
#pragma unroll
      for (int e = 0; e < 16; e++) mx = fmaxf(mx, sacc[1][e]);
      mx = max_halves(mx);
      const float m_new = fmaxf(m_used, mx);
      const bool grow = (m_new - m_used) * c > kLazyRescaleLog2;  // true on the first tile (-inf)
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float alpha = fast_exp2((m_used - m_new) * c);  // 0 on the first tile
        m_used = m_new;
        l_part *= alpha;
#pragma unroll
        for (int db = 0; db < DBLOCKS; db++)
#pragma unroll
          for (int e = 0; e < 16; e++) oacc[db][e] *= alpha;
      }
      const float mc = m_used * c;
      vec8 pf[4];  // P^T as B operands: pf[j] = keys 16j..16j+15 of this tile (permuted inside)
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
          float p0 = fast_exp2(__builtin_fmaf(sacc[kb][e], c, -mc));
          float p1 = fast_exp2(__builtin_fmaf(sacc[kb][e + 1], c, -mc));
          l_part += p0 + p1;
          f32x2 pp = {p0, p1};
          vec2 pk = __builtin_convertvector(pp, vec2);
          const int j = 2 * kb + (e >> 3);
          pf[j][(e & 7)] = pk[0];
          pf[j][(e & 7) + 1] = pk[1];
        }
      }

      // ---- O^T += V^T P^T ------------------------------------------------------------------
      {
        constexpr int PD = kPrefetch;  // MFMAs whose two V^T reads are in flight
        constexpr int NM = 4 * DBLOCKS;
        typedef __attribute__((ext_vector_type(8))) short s16x8;
        s16x4 v0[NM], v1[NM];
        static_for<PD>([&](auto I) {
          constexpr int i_ = I;
          constexpr int off = (i_ / DBLOCKS) * V_J_STEP + (i_ % DBLOCKS) * 64;
          lds_read_tr16_b64<off>(v0[i_], vaddr);
          lds_read_tr16_b64<off + V_RD_STEP>(v1[i_], vaddr);
        });
        static_for<NM>([&](auto I) {
          constexpr int i_ = I;
          constexpr int younger = 2 * ((i_ + PD <= NM ? PD : NM - i_) - 1);
          lds_wait2<younger>(v0[i_], v1[i_]);
          s16x8 vv = __builtin_shufflevector(v0[i_], v1[i_], 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[i_ % DBLOCKS] = Mfma16<T>::mma(__builtin_bit_cast(vec8, vv), pf[i_ / DBLOCKS], oacc[i_ % DBLOCKS]);
          if constexpr (i_ + PD >= NM && i_ + 1 < NM) __builtin_amdgcn_sched_barrier(0);
          if constexpr (i_ + PD < NM) {
            constexpr int n = i_ + PD;
            constexpr int off = (n / DBLOCKS) * V_J_STEP + (n % DBLOCKS) * 64;
            lds_read_tr16_b64<off>(v0[n], vaddr);
            lds_read_tr16_b64<off + V_RD_STEP>(v1[n], vaddr);
          }
        });
      }
      if (drawing && wave == 0 && lane_now() == 0) {
        const bool in_pool = draw < (unsigned)pool_len;
        drawn[i & 1] = in_pool ? seg.pool0 + (int)draw : -1;   // position i + 2
        pool_open = in_pool;
      }
      if (t_next < 0) break;
      t = t_next;
    }
    XDIT_TRACE_POINT(seg.slot >= 0, 2);
    asm volatile("" : "+s"(pp));  // from here on the kernel arguments are read afresh

    // ---- what comes next for this workgroup --------------------------------------------------
    Segment next_seg;
    bool more;
    {
      const WalkGeom g = walk_geom(pp);
      unsigned* const range_counter = pp->split_counter;
      if (walk.wants_claim(range_counter != nullptr && g.split_dyn == 0)) {
        __syncthreads();  // everyone has read the ticket of the previous claim
        if (wave == 0 && lane_now() == 0) ticket = atomicAdd(range_counter, 1u);
        __syncthreads();
        walk.claimed(g, (unsigned)__builtin_amdgcn_readfirstlane((int)ticket));
      }
      more = walk.next(g, nt, next_seg);
    }
    __syncthreads();  // every wavefront is done with the K/V fragments of the last tile
    if (more) {
      XDIT_TRACE_POINT(next_seg.slot >= 0, 0);
      open_segment(next_seg);  // Q fragments and first K/V tile (buffer 0) of the next segment
    }

    // ---- epilogue -----------------------------------------------------------------------------
    const int lane = lane_now(), l32 = lane & 31, hh = lane >> 5;
    const int cqrow = cqt * kRowsPerBlock + wave * kRowsPerWave + l32;
    const float l_tot = sum_halves(l_part);
    const float inv = 1.0f / l_tot;
    const float lse = (m_used * c + fast_log2(l_tot)) * kLn2;
    XDIT_LDS unsigned char* stage = (XDIT_LDS unsigned char*)smem + G::BUF_BYTES + wave * kStageBytes;
    const int row0 = cqt * kRowsPerBlock + wave * kRowsPerWave;   // first query row of this wavefront
    if (!FUSED || part_out != nullptr) {
      // The normalised rows go out through LDS, 64 columns at a time: lane (query, half) writes
      // its 4-element pieces into a [32 rows][64 columns] block private to the wavefront, which is
      // read back with 8 lanes per row, so that every global store covers whole 128-byte lines of
      // 8 rows (stored straight from the accumulator layout, a store touches 32 rows 16 bytes at
      // a time and the epilogue is bound by the number of memory requests).
      typedef __attribute__((ext_vector_type(4))) T vec4;
      T* obase;
      int64_t ostride;
      int rows_live = kRowsPerWave;
      if (part_out != nullptr) {
        obase = part_out + (int64_t)(wave * kRowsPerWave) * D;
        ostride = D;
      } else {
        obase = (T*)pp->out + cb * pp->os_b + ch * pp->os_h + (int64_t)row0 * pp->os_s;
        ostride = pp->os_s;
        rows_live = pp->Sq - row0;  // may be <= 0 or above 32
      }
      const int cols_live = part_out != nullptr ? 32 * DBLOCKS : (PAD ? dact : D);
      const int rd_row = lane >> 3;          // + 8r
      const int rd_col = (lane & 7) * 8;     // element column within the 64-column pass
#pragma unroll
      for (int half = 0; half < (DBLOCKS + 1) / 2; half++) {
#pragma unroll
        for (int dbl = 0; dbl < 2; dbl++) {
          const int db = 2 * half + dbl;
          if (db < DBLOCKS) {
#pragma unroll
            for (int a = 0; a < 4; a++) {
              // registers 4a..4a+3 are d = 32db + 8a + 4hh + 0..3 of this lane's query
              f32x4 o = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv,
                         oacc[db][4 * a + 3] * inv};
              *(XDIT_LDS vec4*)(stage + l32 * kStagePitch + (32 * dbl + 8 * a + 4 * hh) * 2) = __builtin_convertvector(o, vec4);
            }
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int row = rd_row + 8 * r;
          const int col = 64 * half + rd_col;
          const vec8 x = *(const XDIT_LDS vec8*)(stage + row * kStagePitch + rd_col * 2);
          // streaming stores: the rows are not read again by this kernel, and lines that leave the
          // cache as they are written are not left for the write-back at the kernel's end
          if (row < rows_live && col < cols_live) {
            if (FUSED && part_out != nullptr) store16_device(obase + row * ostride + col, __builtin_bit_cast(i32x4, x));  // read by another workgroup of this launch
            else __builtin_nontemporal_store(x, (vec8*)(obase + row * ostride + col));
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
      // Ring step: fold this block into the fp32 accumulator (the arithmetic of the merge kernel
      // on the block rounded to T, so the result equals forward + merge bit for bit).  The block
      // goes through the same LDS transpose as above, so that the accumulator is read and written
      // in whole rows; the weight of each row's fold travels with it.
      typedef __attribute__((ext_vector_type(4))) T vec4;
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
      T* obase = pp->out != nullptr ? (T*)pp->out + cb * pp->os_b + ch * pp->os_h + (int64_t)row0 * pp->os_s : nullptr;
      const int rows_live = pp->Sq - row0;
      const int cols_live = PAD ? dact : D;
      const int rd_row = lane >> 3;
      const int rd_col = (lane & 7) * 8;
#pragma unroll
      for (int half = 0; half < (DBLOCKS + 1) / 2; half++) {
#pragma unroll
        for (int dbl = 0; dbl < 2; dbl++) {
          const int db = 2 * half + dbl;
          if (db < DBLOCKS) {
#pragma unroll
            for (int a = 0; a < 4; a++) {
              f32x4 o = {oacc[db][4 * a] * inv, oacc[db][4 * a + 1] * inv, oacc[db][4 * a + 2] * inv,
                         oacc[db][4 * a + 3] * inv};
              *(XDIT_LDS vec4*)(stage + l32 * kStagePitch + (32 * dbl + 8 * a + 4 * hh) * 2) = __builtin_convertvector(o, vec4);
            }
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
          if (row < rows_live && col < cols_live) {
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
              for (int e = 0; e < 4; e++) { y[e] = (T)m0[e]; y[4 + e] = (T)m1[e]; }
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
    XDIT_TRACE_POINT(seg.slot >= 0, 3);
    if constexpr (FUSED && NW != 12) if (seg.slot >= 0 && pp->split_fold != 0) {
      // this part of a shared tile is written: its arrival, with its fold duty unless that waits for the workgroup's end
      const WalkGeom g = walk_geom(pp);
      const int r = seg.tile - g.split_full;
      const int j = (int)(seg.slot - (int64_t)r * g.split_pmax);
      const int n = shared_tile_parts(g, nt, r);
      const bool now = g.split_order == 0;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's rows of the partial result have been written through
      fold_arrival<T, D, kRowsPerBlock, FUSED>(pp, nt, r, j, n, now, &fold_post);
    }
    if (!more) break;
    if (PAD) {
      // The staging blocks lay over the second K/V buffer: clear it again.  The clearing is striped over the whole
      // buffer, so every wavefront must be done with its staging block first; the barrier of the next segment's first
      // iteration orders the clearing against that segment's tile loads.
      __syncthreads();
      typedef __attribute__((ext_vector_type(4))) int i32x4;
      const i32x4 zero = {0, 0, 0, 0};
      for (int i = (wave * 64 + lane) * 16; i < G::BUF_BYTES; i += 64 * kWaves * 16) *(XDIT_LDS i32x4*)((XDIT_LDS unsigned char*)smem + G::BUF_BYTES + i) = zero;
    }
    seg = next_seg;
  }
  if constexpr (FUSED && NW != 12) if (pp->split_fold != 0) {
    if (pp->split_order != 0) fold_duties_at_end<T, D, kRowsPerBlock, FUSED>(pp, nt, &fold_post);
    if (walk.claimer && pp->split_counter != nullptr && pp->split_dyn == 0) claimer_done(pp);
  }
}

template <typename T, int D, int DC, int NW, bool PAD, bool FUSED>
__global__ __launch_bounds__(64 * NW, NW == 12 ? 3 : 2) void attn_fwd_16_kernel(const AttnParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // [K tile | V tile] [K tile | V tile, or output staging]
  attn_workgroup<T, D, DC, NW, PAD, FUSED>(smem);
}

// Workgroups of NW wavefronts resident at once: LDS and registers allow two 4-wavefront
// workgroups per CU, one otherwise.
static int resident_workgroups(int NW, int planned_cus) { return resident_cus(planned_cus) * (NW == 4 ? 2 : 1); }

template <typename T, int D, int DC, int NW, bool PAD, bool FUSED>
static hipError_t launch_kernel(const AttnParams& q, hipStream_t stream) {
  static std::atomic<bool> lds_ready[kMaxDevices];
  constexpr int lds = lds_bytes_16<D, NW>();
  const int slot = current_device_slot();
  if (!lds_ready[slot].load(std::memory_order_relaxed)) {  // > 64 KiB of dynamic LDS must be enabled once per kernel and device
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_16_kernel<T, D, DC, NW, PAD, FUSED>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    lds_ready[slot].store(true, std::memory_order_relaxed);
  }
  hipLaunchKernelGGL((attn_fwd_16_kernel<T, D, DC, NW, PAD, FUSED>), dim3(split_grid(q)), dim3(64 * NW), lds, stream, q);
  return hipSuccess;
}

template <typename T, int D, int NW, bool FUSED>
static hipError_t launch_one(const AttnParams& p, hipStream_t stream) {
  AttnParams q = p;
  constexpr int rows = 32 * NW;
  q.nq_tiles = (p.Sq + rows - 1) / rows;
  q.total_tiles = p.B * p.H * q.nq_tiles;
  q.tiles_per_xcd = (q.total_tiles + 7) / 8;
  // the ring step takes a balanced plan only when the attention kernel folds the parts itself (the fold goes on into the accumulator)
  bind_workspace(q, p, plan_split(q, rows, resident_workgroups(NW, p.cu_count), D, 2, kClaimsPerWorkgroup, true, FUSED), rows, D, 2);
  if (q.d_actual == D) q.d_actual = 0;
  // computed head_dims built for tensors smaller than D: 80, 96, 112 (and 128) of 128; 32 (and 64) of 64
  hipError_t e;
  if (q.d_actual == 0) {
    e = launch_kernel<T, D, D, NW, false, FUSED>(q, stream);
  } else if constexpr (D == 128) {
    e = q.d_actual <= 80    ? launch_kernel<T, D, 80, NW, true, FUSED>(q, stream)
        : q.d_actual <= 96  ? launch_kernel<T, D, 96, NW, true, FUSED>(q, stream)
        : q.d_actual <= 112 ? launch_kernel<T, D, 112, NW, true, FUSED>(q, stream)
                            : launch_kernel<T, D, 128, NW, true, FUSED>(q, stream);
  } else {
    e = q.d_actual <= 32 ? launch_kernel<T, D, 32, NW, true, FUSED>(q, stream) : launch_kernel<T, D, 64, NW, true, FUSED>(q, stream);
  }
  if (e != hipSuccess) return e;
  if constexpr (!FUSED) {
    if (q.split_units && !q.split_fold) {  // tiles of many parts: folded by a launch of its own
      const int nt = (q.Sk + kKeysPerTile - 1) / kKeysPerTile + (q.Sk2 + kKeysPerTile - 1) / kKeysPerTile;
      const dim3 cgrid((unsigned)((rows * (D / 8) + 255) / 256), (unsigned)(q.total_tiles - q.split_full));
      hipLaunchKernelGGL((attn_combine_kernel<T, D>), cgrid, dim3(256), 0, stream, q, rows, nt, split_counters(q));
    }
  }
  return hipGetLastError();
}

// D: the head_dim the kernel is built for, 128 or 64; p.d_actual, if not 0, is the tensors'
// smaller head_dim (a multiple of 8).  rows_per_block: 128 (4 wavefronts), 256 (8) or 384 (12).
// FUSED: the ring step (p.acc_out set), whose epilogue folds the block into the accumulator.
template <typename T, bool FUSED>
static hipError_t launch_typed(const AttnParams& p, int D, int rows_per_block, hipStream_t stream) {
  if (D == 128 && rows_per_block == 384) return launch_one<T, 128, 12, FUSED>(p, stream);
  if (D == 128 && rows_per_block == 256) return launch_one<T, 128, 8, FUSED>(p, stream);
  if (D == 128) return launch_one<T, 128, 4, FUSED>(p, stream);
  if (D == 64 && rows_per_block == 384) return launch_one<T, 64, 12, FUSED>(p, stream);
  if (D == 64 && rows_per_block == 256) return launch_one<T, 64, 8, FUSED>(p, stream);
  if (D == 64) return launch_one<T, 64, 4, FUSED>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace xdit
