// Balanced launch shared by the attention kernels: when the query tiles do not fill a whole
// number of rounds of resident workgroups, the KV iterations of the last round's tiles are cut
// into equal ranges, one per workgroup; partial (out, lse) pairs go through a workspace and are
// folded by attn_combine_kernel.
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
  int total_tiles, tiles_per_xcd, split_full, split_units, split_len, split_pmax, split_fuse0, split_claimers, split_dyn, split_s0;
};
typedef const __attribute__((address_space(4))) AttnParams* ParamsPtr;
__device__ __forceinline__ WalkGeom walk_geom(ParamsPtr pp) {
  WalkGeom g = {pp->total_tiles, pp->tiles_per_xcd, pp->split_full, pp->split_units, pp->split_len, pp->split_pmax,
                pp->split_fuse0, pp->split_claimers, pp->split_dyn, pp->split_s0};
  return g;
}

// Runs the segments of this workgroup (see WorkgroupWalk in attn_walk.h for who does what).
// `seg(tile, it0, it1, part_out, part_lse)` processes KV tiles [it0, it1) of query tile `tile`;
// part_out == nullptr means "write the final result", otherwise the normalised partial result and
// its log-sum-exp go to that workspace slot.  TO is the output element type, ROWS the query rows
// per workgroup.
template <typename TO, int ROWS, int D, typename Seg>
__device__ __forceinline__ void run_workgroup(const AttnParams& p, Seg seg) {
  const int nt = (p.Sk + kKeysPerTile - 1) / kKeysPerTile + (p.Sk2 + kKeysPerTile - 1) / kKeysPerTile;
  __shared__ unsigned ticket;
  WorkgroupWalk walk;
  if (!walk.start(p, nt, (int)blockIdx.x)) return;
  bool first = true;
  Segment s;
  while (walk.next(p, nt, s)) {  // one segment per turn; a single call site keeps one copy of the kernel body
    TO* part_out = nullptr;
    float* part_lse = nullptr;
    if (s.slot >= 0) {
      part_out = (TO*)p.ws_out + s.slot * ROWS * D;
      part_lse = p.ws_lse + s.slot * ROWS;
    }
    if (!first) __syncthreads();  // every wavefront is done with the LDS buffers of the previous segment
    seg(s.tile, s.it0, s.it1, part_out, part_lse);
    first = false;
    if (walk.wants_claim(p.split_counter != nullptr)) {
      __syncthreads();  // everyone has read the ticket of the previous claim
      if (threadIdx.x == 0) ticket = atomicAdd(p.split_counter, 1u);
      __syncthreads();
      walk.claimed(p, ticket);
    }
  }
}

// Clears the counters of a balanced launch (a kernel, not a memset, so that the sequence can be
// captured into a graph).
static __global__ void attn_counter_reset_kernel(unsigned* counter, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) counter[i] = 0u;
}

// Folds the parts of every query tile that was split: out = sum_k exp(lse_k - L) out_k,
// L = log sum_k exp(lse_k), in fp32; one thread per 8 head_dim elements of a row.
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
  // One pass, eight parts in flight per thread (outputs and log-sum-exps are loaded together,
  // so a tile of up to eight parts costs one round trip to memory); the running maximum L is
  // carried from one group of eight to the next as in the online softmax.
  float L = -INFINITY;
  float denom = 0.f;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < nparts; k0 += 8) {
    vec8 x[8];
    float ls[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int k = k0 + j < nparts ? k0 + j : nparts - 1;
      x[j] = *(const vec8*)(part0 + (int64_t)k * rows_per_block * D);
      ls[j] = lsep[(int64_t)k * rows_per_block];
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
  vec8 o;
#pragma unroll
  for (int i = 0; i < 8; i++) o[i] = (T)(acc[i] * inv);
  *(vec8*)((T*)p.out + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_s + col) = o;
  if (col == 0 && p.lse != nullptr) p.lse[b * p.ls_b + h * p.ls_h + qrow] = L + __logf(denom);
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

static inline size_t plan_split(AttnParams& q, int rows, int slots, int D, int out_bytes, int claims, bool streamed = false) {
  q.split_units = q.split_full = q.split_len = q.split_pmax = q.split_share = q.split_claimers = 0;
  q.split_fuse0 = 0x7fffffff;
  q.split_counter = nullptr;
  q.split_dyn = q.split_s0 = 0;
  const int nt = (q.Sk + kKeysPerTile - 1) / kKeysPerTile + (q.Sk2 + kKeysPerTile - 1) / kKeysPerTile;
  const int T = q.total_tiles;
  const int full = (T / slots) * slots;
  const int rem = T - full;
  if (rem == 0 || nt < 8) return 0;
  int share = (int)(((int64_t)rem * nt + slots - 1) / slots);  // iterations per workgroup
  if (share < 4) share = 4;
  // Iterations of the critical path saved by filling the last round: a plan is offered when it
  // saves at least kMinSaving of them; whether it is taken is the caller's decision (the time
  // estimate of the C entry points compares it with the plain launch; split_policy 1 refuses it).
  if (q.split_policy == 1 || nt - share < kMinSaving) return 0;
  // Few shared tiles with short shares: streamed sharing.  Every resident workgroup joins the
  // group of one shared tile; unless the caller asks for bit-reproducible results.
  if (streamed && !q.deterministic && share < 2 * kMinClaimLen && rem * 4 <= slots) {
    const int pmax = (slots + rem - 1) / rem;
    if (pmax * kStreamedOwn * 2 <= nt && (size_t)rem * 4 <= kCounterRegionBytes) {
      q.split_full = full;
      q.split_units = q.split_claimers = slots;
      q.split_len = share;
      q.split_share = share;
      q.split_pmax = pmax;
      q.split_fuse0 = full >= slots ? full - slots : 0x7fffffff;
      q.split_dyn = 1;
      q.split_s0 = kStreamedOwn;
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
  return kCounterRegionBytes + split_parts_bytes(q, rows, D, out_bytes);
}

// Lay the workspace out: counters, partial outputs, partial log-sum-exps; or fall back to a plain
// launch when the caller gave no (or too small a) workspace.
static inline void bind_workspace(AttnParams& q, const AttnParams& p, size_t need, int rows, int D, int out_bytes) {
  if (need == 0 || p.ws_out == nullptr || p.ws_bytes < need) {
    q.split_units = q.split_full = q.split_len = q.split_pmax = q.split_share = q.split_claimers = 0;
    q.split_fuse0 = 0x7fffffff;
    q.split_counter = nullptr;
    q.split_dyn = q.split_s0 = 0;
    q.ws_out = nullptr;
  } else {
    const size_t rem = (size_t)(q.total_tiles - q.split_full);
    q.ws_counters = (unsigned*)p.ws_out;
    q.ws_out = (unsigned char*)p.ws_out + kCounterRegionBytes;
    q.ws_lse = (float*)((unsigned char*)q.ws_out + rem * q.split_pmax * rows * D * out_bytes);
    q.split_counter = split_counters(q) > 0 ? q.ws_counters : nullptr;
  }
}

// The launches around the attention kernel of a balanced launch.  Counters must be zero when the
// attention kernel starts: a workspace whose contents the caller vouches for (ws_preserved: left
// as this library's previous call on it left them) has them at zero already, since the fold
// kernel clears what its launch used; otherwise a small kernel clears the whole region first.
static inline void launch_counter_reset(const AttnParams& q, hipStream_t stream) {
  if (q.split_units != 0 && !q.ws_preserved)
    hipLaunchKernelGGL(attn_counter_reset_kernel, dim3(1), dim3(256), 0, stream, q.ws_counters, (int)(kCounterRegionBytes / 4));
}

// Workgroups of a launch planned by plan_split (after bind_workspace).
static inline unsigned split_grid(const AttnParams& q) {
  if (q.split_units == 0) return (unsigned)(q.tiles_per_xcd * 8);
  return (unsigned)(q.split_fuse0 <= q.split_full ? q.split_full : q.split_full + q.split_claimers);
}

}  // namespace xdit
