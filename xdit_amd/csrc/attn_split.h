// Balanced launch shared by the attention kernels: when the query tiles do not fill a whole
// number of rounds of resident workgroups, the KV iterations of the last round's tiles are cut
// into equal ranges, one per workgroup; partial (out, lse) pairs go through a workspace and are
// folded by the workgroups of the attention kernel themselves (fold duties) or, for tiles of many
// parts, by attn_combine_kernel.
#pragma once
#include <atomic>

#include "attn_tiles.h"

namespace xdit {

// The lane's index within its wavefront, computed where it is called (two instructions) instead
// of being kept in a register through the KV loop; not merged with other calls by the compiler.
__device__ __forceinline__ int lane_now() {
  int x;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(x));
  return x;
}

// One ticket from a counter in device memory (device-scope atomic add of 1, relaxed), for a branch
// that a single lane takes.  The operands are formed right here rather than kept in registers
// through the KV loop around it.
__device__ __forceinline__ unsigned draw_ticket(unsigned* counter) {
  unsigned one = 1;
  asm volatile("" : "+v"(one));
  return __hip_atomic_fetch_add(counter, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The launch geometry the walker reads, gathered from the kernel arguments when needed.
struct WalkGeom {
  int total_tiles, tiles_per_xcd, split_full, split_units, split_len, split_pmax, split_fuse0, split_claimers, split_dyn, split_s0, split_order;
};
typedef const __attribute__((address_space(4))) AttnParams* ParamsPtr;
__device__ __forceinline__ WalkGeom walk_geom(ParamsPtr pp) {
  WalkGeom g = {pp->total_tiles, pp->tiles_per_xcd, pp->split_full, pp->split_units, pp->split_len, pp->split_pmax,
                pp->split_fuse0, pp->split_claimers, pp->split_dyn, pp->split_s0, pp->split_order};
  return g;
}

// Clears the counters of a balanced launch (a kernel, not a memset, so that the sequence can be
// captured into a graph).
static __global__ void attn_counter_reset_kernel(unsigned* counter, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) counter[i] = 0u;
}

// Partial results that are folded inside the same launch cross from one XCD to another, whose L2
// caches are not coherent with each other for ordinary accesses.  They are therefore written and
// read with device-scope (relaxed atomic) accesses of 8 bytes, which the L2 passes through to
// memory, instead of ordinary accesses bracketed by device-scope fences: such a fence writes back
// (release) or invalidates (acquire) the whole L2 of the XCD, which cost the Flux step 30-45 us.
// Order is kept by hand: a wavefront waits for its stores to complete (s_waitcnt vmcnt(0)) before
// the workgroup barrier that precedes the arrival's atomic add, and the loads are issued after the
// barrier that follows it.
__device__ __forceinline__ void store16_device(void* p, i32x4 x) {
  unsigned long long lo = ((unsigned long long)(unsigned)x[1] << 32) | (unsigned)x[0];
  unsigned long long hi = ((unsigned long long)(unsigned)x[3] << 32) | (unsigned)x[2];
  __hip_atomic_store((unsigned long long*)p, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store((unsigned long long*)p + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ i32x4 load16_device(const void* p) {
  const unsigned long long lo = __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long hi = __hip_atomic_load((const unsigned long long*)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  i32x4 x = {(int)(unsigned)lo, (int)(unsigned)(lo >> 32), (int)(unsigned)hi, (int)(unsigned)(hi >> 32)};
  return x;
}
__device__ __forceinline__ void store_float_device(float* p, float x) { __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float load_float_device(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// One (row, 8-column chunk) of a shared query tile folded from its parts:
//   out = sum_k exp(lse_k - L) out_k / sum_k exp(lse_k - L),  lse = L + log sum_k exp(lse_k - L),  L = max_k lse_k,
// in fp32, the parts taken in slot order.  `part0` / `lsep` point at this chunk / row in part 0;
// parts are `out_stride` elements / `lse_stride` floats apart.  Eight parts are in flight per
// thread (outputs and log-sum-exps loaded together, so a tile of up to eight parts costs one round
// trip to memory); the running maximum L is carried from one group of eight to the next as in the
// online softmax.  Used by attn_combine_kernel and by the fold inside the attention kernels, so
// that both give the same bits.  DEVICE: the parts were written by other workgroups of this launch
// (device-scope loads, see above).
template <typename T, bool DEVICE>
__device__ __forceinline__ void combine_item(const T* part0, const float* lsep, int nparts, int64_t out_stride, int64_t lse_stride,
                                             __attribute__((ext_vector_type(8))) T& o, float& lse_out) {
  typedef __attribute__((ext_vector_type(8))) T vec8;
  float L = -INFINITY;
  float denom = 0.f;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < nparts; k0 += 8) {
    vec8 x[8];
    float ls[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int k = k0 + j < nparts ? k0 + j : nparts - 1;
      if constexpr (DEVICE) {
        x[j] = __builtin_bit_cast(vec8, load16_device(part0 + (int64_t)k * out_stride));
        ls[j] = load_float_device(lsep + (int64_t)k * lse_stride);
      } else {
        x[j] = *(const vec8*)(part0 + (int64_t)k * out_stride);
        ls[j] = lsep[(int64_t)k * lse_stride];
      }
    }
    float Ln = L;
#pragma unroll
    for (int j = 0; j < 8; j++) Ln = fmaxf(Ln, ls[j]);
    const float keep = __expf(L - Ln);  // 0 on the first group (L = -inf)
    L = Ln;
    denom *= keep;
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] *= keep;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float w = k0 + j < nparts ? __expf(ls[j] - L) : 0.f;
      denom += w;
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i] += w * (float)x[j][i];
    }
  }
  const float inv = 1.0f / denom;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    // the product is rounded to fp32 and THEN to T wherever this is inlined: left alone, the compiler
    // takes a multiply that rounds straight to fp16 in some contexts and not in others (one unit in
    // the last place apart in about one element of 10^4)
    float t = acc[i] * inv;
    asm volatile("" : "+v"(t));
    o[i] = (T)t;
  }
  lse_out = L + __logf(denom);
}

// Folds the parts of every query tile that was split (launches whose tiles have more parts than
// the attention kernel folds itself); one thread per 8 head_dim elements of a row.
// grid = (ceil(rows_per_block * D/8 / 256), shared query tiles): blockIdx.y is the tile, so the
// tile's coordinates and part range are wavefront-uniform.
template <typename T, int D>
__global__ __launch_bounds__(256) void attn_combine_kernel(const AttnParams p, const int rows_per_block, const int nt, const int counters) {
  constexpr int TPR = D / 8;
  const int r = blockIdx.y;  // which of the shared query tiles
  const int local = blockIdx.x * 256 + threadIdx.x;
  // the counters the attention kernel used go back to zero, for the next call on this workspace
  if (blockIdx.x == 0 && blockIdx.y == 0)
    for (int i = threadIdx.x; i < counters; i += 256) p.ws_counters[i] = 0u;
  const int row = local / TPR;
  const int col = (local - row * TPR) * 8;
  if (row >= rows_per_block) return;
  if (p.d_actual != 0 && col >= p.d_actual) return;  // columns the tensors do not have
  const int tile = p.split_full + r;
  const int bh = tile / p.nq_tiles;
  const int qt = tile - bh * p.nq_tiles;
  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int qrow = qt * rows_per_block + row;
  if (qrow >= p.Sq) return;
  const int nparts = shared_tile_parts(p, nt, r);
  const float* lsep = p.ws_lse + ((int64_t)r * p.split_pmax) * rows_per_block + row;
  typedef __attribute__((ext_vector_type(8))) T vec8;
  const T* part0 = (const T*)p.ws_out + (((int64_t)r * p.split_pmax) * rows_per_block + row) * D + col;
  vec8 o;
  float lse;
  combine_item<T, false>(part0, lsep, nparts, (int64_t)rows_per_block * D, rows_per_block, o, lse);
  *(vec8*)((T*)p.out + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_s + col) = o;
  if (col == 0 && p.lse != nullptr) p.lse[b * p.ls_b + h * p.ls_h + qrow] = lse;
}

// ---- the fold inside the attention kernels (fold duties, see attn_walk.h) ----------------------
// Counter region of a workspace (4096 words): [0, kArriveBase) the range counter of a launch or
// the per-tile counters of streamed sharing; [kArriveBase, kDoneIndex) one fold word per shared
// tile; kDoneIndex counts the claimers that have finished (its last one clears the range counter).
constexpr int kArriveBase = 2048;
constexpr int kDoneIndex = 4095;

// Rows of shared tile r (the slices in `mask`, n parts) folded by all threads of the workgroup and
// written to the output tensors, or, FUSED (the ring step), folded further into the fp32
// accumulator with the arithmetic of the merge kernel on the folded block rounded to T.  The
// D/8 chunks of a row are held by adjacent lanes of one wavefront in the same pass, so every lane
// of a row has read the accumulated log-sum-exp before the row's first lane overwrites it.
template <typename T, int D, int ROWS, bool FUSED>
__device__ __forceinline__ void fold_tile_slices(ParamsPtr pp, int nt, int r, unsigned mask, int n) {
  constexpr int TPR = D / 8;
  typedef __attribute__((ext_vector_type(8))) T vec8;
  const int tid = (int)threadIdx.x, nthreads = (int)blockDim.x;
  const int nq_tiles = pp->nq_tiles, H = pp->H, Sq = pp->Sq, dact = pp->d_actual, pmax = pp->split_pmax;
  const int tile = pp->split_full + r;
  const int bh = tile / nq_tiles;
  const int qt = tile - bh * nq_tiles;
  const int b = bh / H;
  const int h = bh - b * H;
  const T* const parts = (const T*)pp->ws_out + ((int64_t)r * pmax) * ROWS * D;
  const float* const lses = pp->ws_lse + ((int64_t)r * pmax) * ROWS;
  const bool all = mask == (n >= 32 ? 0xffffffffu : (1u << n) - 1u);
  for (int j = 0; j < n; j++) {
    int r0 = 0, r1 = ROWS;
    if (!all) {
      if (!((mask >> j) & 1u)) continue;
      fold_slice_rows(j, n, ROWS, r0, r1);
    }
    for (int item = tid; item < (r1 - r0) * TPR; item += nthreads) {
      const int row = r0 + item / TPR;
      const int col = (item % TPR) * 8;
      const int qrow = qt * ROWS + row;
      if (qrow >= Sq || (dact != 0 && col >= dact)) continue;
      vec8 o;
      float lse;
      combine_item<T, true>(parts + (int64_t)row * D + col, lses + row, n, (int64_t)ROWS * D, ROWS, o, lse);
      if constexpr (!FUSED) {
        *(vec8*)((T*)pp->out + b * pp->os_b + h * pp->os_h + (int64_t)qrow * pp->os_s + col) = o;
        if (col == 0 && pp->lse != nullptr) pp->lse[b * pp->ls_b + h * pp->ls_h + qrow] = lse;
      } else {
        const bool first = pp->acc_first != 0;
        float* alp = pp->acc_lse + b * pp->al_b + h * pp->al_h + (int64_t)qrow * pp->al_s;
        float* aptr = pp->acc_out + b * pp->ao_b + h * pp->ao_h + (int64_t)qrow * pp->ao_s + col;
        f32x4 m0, m1;
#pragma unroll
        for (int e = 0; e < 4; e++) { m0[e] = (float)o[e]; m1[e] = (float)o[4 + e]; }
        float new_lse = lse;
        if (!first) {
          const float la = *alp;  // read by every lane of the row before its first lane stores below
          const float w = sigmoid(lse - la);
          new_lse = la - log_sigmoid(la - lse);
          const f32x4 a0 = *(const f32x4*)aptr, a1 = *(const f32x4*)(aptr + 4);
#pragma unroll
          for (int e = 0; e < 4; e++) { m0[e] = fold_value(a0[e], m0[e], w); m1[e] = fold_value(a1[e], m1[e], w); }
        }
        if (pp->acc_store) { *(f32x4*)aptr = m0; *(f32x4*)(aptr + 4) = m1; }
        if (pp->out != nullptr) {
          vec8 y;
#pragma unroll
          for (int e = 0; e < 4; e++) { y[e] = (T)m0[e]; y[4 + e] = (T)m1[e]; }
          *(vec8*)((T*)pp->out + b * pp->os_b + h * pp->os_h + (int64_t)qrow * pp->os_s + col) = y;
        }
        if (col == 0) {
          *alp = new_lse;
          if (pp->lse != nullptr) pp->lse[b * pp->ls_b + h * pp->ls_h + qrow] = new_lse;
        }
      }
    }
    if (all) break;
  }
}

// One event on the fold word of shared tile r by this workgroup (every thread calls it):
// `arrival`: part j of the tile's n parts has just been written by this workgroup (with_duty: its
// fold duty is presented with it); otherwise the duty of part j is presented on its own.  Folds
// what the protocol hands this workgroup.  `post` is one word of LDS.
template <typename T, int D, int ROWS, bool FUSED>
__device__ __forceinline__ void fold_event_body(ParamsPtr pp, int nt, int r, int j, int n, bool arrival, bool with_duty, unsigned* post) {
  __syncthreads();  // every wavefront's rows of the partial result have been stored (and awaited by it); `post` is free
  if (threadIdx.x == 0) {
    unsigned* const word = pp->ws_counters + kArriveBase + r;
    const unsigned add = arrival ? fold_arrive_word(j, with_duty) : fold_duty_word(j);
    const unsigned old = __hip_atomic_fetch_add(word, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (fold_last_event(old, add, n)) {  // nobody touches the tile's counters after this event
      __hip_atomic_store(word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (pp->split_dyn) __hip_atomic_store(pp->ws_counters + r, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    *post = arrival ? fold_after_arrival(old, j, with_duty, n) : fold_after_duty(old, j, n);
  }
  __syncthreads();
  const unsigned mask = (unsigned)__builtin_amdgcn_readfirstlane((int)*post);
  if (mask != 0u) {
    fold_tile_slices<T, D, ROWS, FUSED>(pp, nt, r, mask, n);
  }
}

// The arrival of part j of shared tile r, called by the attention kernels after the part's rows are
// stored.
template <typename T, int D, int ROWS, bool FUSED>
__device__ __forceinline__ void fold_arrival(ParamsPtr pp, int nt, int r, int j, int n, bool with_duty, unsigned* post) {
  fold_event_body<T, D, ROWS, FUSED>(pp, nt, r, j, n, true, with_duty, post);
}

// At the very end of a workgroup of a parts-first launch: the fold duties of the parts it wrote at
// its start.  Claimer c = workgroup split_fuse0 + c of such a launch has range c, whose (up to
// two) parts are worked out again here rather than carried through the KV loops.
template <typename T, int D, int ROWS, bool FUSED>
__device__ __forceinline__ void fold_duties_at_end(ParamsPtr pp, int nt, unsigned* post) {
  const WalkGeom g = walk_geom(pp);
  const int u = (int)blockIdx.x - g.split_fuse0;
  if (u < 0 || u >= g.split_units) return;
  const int rem_iters = (g.total_tiles - g.split_full) * nt;
  int lin = u * g.split_len;
  const int lin_end = lin + g.split_len < rem_iters ? lin + g.split_len : rem_iters;
  while (lin < lin_end) {
    const int r = lin / nt;
    const int it1 = lin_end - r * nt < nt ? lin_end - r * nt : nt;
    const int j = u - (r * nt) / g.split_len;
    fold_event_body<T, D, ROWS, FUSED>(pp, nt, r, j, shared_tile_parts(g, nt, r), false, false, post);
    lin = r * nt + it1;
  }
}

// At the very end of a claimer of a launch that hands ranges out through a counter and folds in
// the kernel: the last claimer to finish puts the range counter (and this count) back to zero.
__device__ __forceinline__ void claimer_done(ParamsPtr pp) {
  if (threadIdx.x == 0) {
    unsigned* const done = pp->ws_counters + kDoneIndex;
    const unsigned old = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((int)old == pp->split_claimers - 1) {
      __hip_atomic_store(done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(pp->ws_counters, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// State cached per device (a process may drive several): index of the current device.
constexpr int kMaxDevices = 64;
static inline int current_device_slot() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = 0;
  return dev % kMaxDevices;
}

// Compute units of the current device (cached; concurrent first calls store the same value), or
// the number the caller plans for.
static inline int resident_cus(int planned = 0) {
  if (planned > 0) return planned;
  static std::atomic<int> cus[kMaxDevices];
  const int slot = current_device_slot();
  int n = cus[slot].load(std::memory_order_relaxed);
  if (n == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[slot].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Ranges shorter than this many KV iterations are not worth a claim of their own (prologue,
// epilogue and partial result of a segment cost about four iterations).
constexpr int kMinClaimLen = 64;
// Ranges per claimer aimed at when ranges are claimed one after the other.  Worth it for the
// 16-bit kernels, which run power-limited with XCD clocks several per cent apart (HunyuanVideo
// shard: 18.22 -> 17.85 ms at 6, 17.95 at 4 and at 12); the fp8 kernel runs at equal clocks and
// only pays for the extra partial results.
constexpr int kClaimsPerWorkgroup = 6;

// Decide how to balance the launch; fills the split_* fields of q.  Returns the workspace bytes
// the balanced launch needs (0 = plain launch).
// `rows` query rows per workgroup, `slots` workgroups resident at once, `out_bytes` per output
// element, `claims` ranges per workgroup to aim at (1: every workgroup gets one range).
// A workspace starts with this many bytes of counters (4096 of them), whatever the launch uses of
// them: partial results never lie there, so counters that one call leaves at zero are still zero
// for the next call on the same workspace, whatever its shape.
constexpr size_t kCounterRegionBytes = 16384;

// Fewest KV iterations of critical path a balanced launch must save to be offered at all.
constexpr int kMinSaving = 12;

// Iterations a member of a tile's group owns under streamed sharing (the loop needs two to start
// drawing from the counter without waiting for it).
constexpr int kStreamedOwn = 2;

// Number of counters a planned launch uses (0: none).
static inline int split_counters(const AttnParams& q) {
  if (q.split_dyn) return q.total_tiles - q.split_full;
  return q.split_units > q.split_claimers ? 1 : 0;
}
static inline size_t split_parts_bytes(const AttnParams& q, int rows, int D, int out_bytes) {
  return (size_t)(q.total_tiles - q.split_full) * q.split_pmax * rows * ((size_t)D * out_bytes + 4);
}

// The ring step folds the parts of its shared tiles inside the attention kernel (fold duties,
// attn_walk.h: its fold goes on into the accumulator), which takes tiles of few parts; a plain
// forward leaves them to attn_combine_kernel, a launch of its own (measured on Flux-1024 and on
// three of its heads the fold inside the kernel was 6-8 % slower: whoever folds a tile reads all
// of its parts alone, one round trip to memory after the other, at the very end of the launch).
// Also whether the claimers take their range before their whole tile (possible when every claimer
// has exactly one range and a whole tile; the parts are then complete long before the workgroups
// end, and each folds its slice there instead of the last one folding everything).
static inline void plan_fold(AttnParams& q) {
  const int rem = q.total_tiles - q.split_full;
  q.split_fold = q.split_units != 0 && q.split_pmax <= kFoldMaxParts && rem < kDoneIndex - kArriveBase ? 1 : 0;
  q.split_order = q.split_fold && !q.split_dyn && q.split_units <= q.split_claimers && q.split_fuse0 <= q.split_full ? 1 : 0;
}

// `fold_only`: offer a plan only if the attention kernel folds the parts itself (the ring step,
// whose fold goes on into the accumulator).
static inline size_t plan_split(AttnParams& q, int rows, int slots, int D, int out_bytes, int claims, bool streamed = false, bool fold_only = false) {
  q.split_units = q.split_full = q.split_len = q.split_pmax = q.split_share = q.split_claimers = 0;
  q.split_fuse0 = 0x7fffffff;
  q.split_counter = nullptr;
  q.split_dyn = q.split_s0 = q.split_order = q.split_fold = 0;
  const int nt = (q.Sk + kKeysPerTile - 1) / kKeysPerTile + (q.Sk2 + kKeysPerTile - 1) / kKeysPerTile;
  const int T = q.total_tiles;
  const int full = (T / slots) * slots;
  const int rem = T - full;
  if (rem == 0 || nt < 8) return 0;
  if (fold_only && rows > 256) return 0;  // the 12-wavefront ring-step kernels have no registers to spare for the fold
  int share = (int)(((int64_t)rem * nt + slots - 1) / slots);  // iterations per workgroup
  if (share < 4) share = 4;
  // Iterations of the critical path saved by filling the last round: a plan is offered when it
  // saves at least kMinSaving of them; whether it is taken is the caller's decision (the time
  // estimate of the C entry points compares it with the plain launch; split_policy 1 refuses it).
  if (q.split_policy == 1 || nt - share < kMinSaving) return 0;
  // Few shared tiles with short shares: streamed sharing.  Every resident workgroup joins the
  // group of one shared tile; unless the caller asks for bit-reproducible results.
  if (streamed && q.streamed_ok && share < 2 * kMinClaimLen && rem * 4 <= slots) {
    const int pmax = (slots + rem - 1) / rem;
    if (pmax * kStreamedOwn * 2 <= nt && rem <= kArriveBase && (!fold_only || pmax <= kFoldMaxParts)) {
      q.split_full = full;
      q.split_units = q.split_claimers = slots;
      q.split_len = share;
      q.split_share = share;
      q.split_pmax = pmax;
      q.split_fuse0 = full >= slots ? full - slots : 0x7fffffff;
      q.split_dyn = 1;
      q.split_s0 = kStreamedOwn;
      if (fold_only) plan_fold(q);
      return kCounterRegionBytes + split_parts_bytes(q, rows, D, out_bytes);
    }
  }
  // Long shares are cut into several ranges that are claimed one after the other: as many per
  // claimer as the minimum range length allows, up to `claims`, and of a length that gives every
  // claimer that whole number of ranges (2.25 ranges per claimer would end with a quarter of the
  // compute units running a third range alone).
  int len = share;
  if (claims > 1 && share >= 2 * kMinClaimLen) {
    const int per_claimer = share / kMinClaimLen < claims ? share / kMinClaimLen : claims;
    len = (share + per_claimer - 1) / per_claimer;
  }
  const int units = (int)(((int64_t)rem * nt + len - 1) / len);
  const int claimers = units < slots ? units : slots;
  q.split_full = full;
  q.split_units = units;
  q.split_len = len;
  q.split_share = share;
  q.split_pmax = (nt + len - 1) / len + 1;
  q.split_claimers = claimers;
  q.split_fuse0 = full >= claimers ? full - claimers : 0x7fffffff;
  if (fold_only) plan_fold(q);
  if (fold_only && !q.split_fold) {
    q.split_units = q.split_full = q.split_len = q.split_pmax = q.split_share = q.split_claimers = 0;
    q.split_fuse0 = 0x7fffffff;
    return 0;
  }
  return kCounterRegionBytes + split_parts_bytes(q, rows, D, out_bytes);
}

// Lay the workspace out: counters, partial outputs, partial log-sum-exps; or fall back to a plain
// launch when the caller gave no (or too small a) workspace.
static inline void bind_workspace(AttnParams& q, const AttnParams& p, size_t need, int rows, int D, int out_bytes) {
  if (need == 0 || p.ws_out == nullptr || p.ws_bytes < need) {
    q.split_units = q.split_full = q.split_len = q.split_pmax = q.split_share = q.split_claimers = 0;
    q.split_fuse0 = 0x7fffffff;
    q.split_counter = nullptr;
    q.split_dyn = q.split_s0 = q.split_order = q.split_fold = 0;
    q.ws_out = nullptr;
  } else {
    const size_t rem = (size_t)(q.total_tiles - q.split_full);
    q.ws_counters = (unsigned*)p.ws_out;
    q.ws_out = (unsigned char*)p.ws_out + kCounterRegionBytes;
    q.ws_lse = (float*)((unsigned char*)q.ws_out + rem * q.split_pmax * rows * D * out_bytes);
    q.split_counter = split_counters(q) > 0 ? q.ws_counters : nullptr;
  }
}

// Clears the counter region of a workspace whose contents the caller does not vouch for.  Done by
// the C entry points for EVERY call that is given such a workspace, balanced or not, so that
// "preserved" means the same whatever the earlier calls on the workspace were.
static inline void launch_counter_reset(void* workspace, hipStream_t stream) {
  hipLaunchKernelGGL(attn_counter_reset_kernel, dim3(1), dim3(256), 0, stream, (unsigned*)workspace, (int)(kCounterRegionBytes / 4));
}

// Workgroups of a launch planned by plan_split (after bind_workspace).
static inline unsigned split_grid(const AttnParams& q) {
  if (q.split_units == 0) return (unsigned)(q.tiles_per_xcd * 8);
  return (unsigned)(q.split_fuse0 <= q.split_full ? q.split_full : q.split_full + q.split_claimers);
}

}  // namespace xdit
