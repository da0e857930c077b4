// C ABI of the attention hot path: argument validation, kernel selection, launch.
// Nothing here allocates device memory or synchronises; every launch goes to the caller's stream.
#include "../../include/xdit_amd_attn.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "attn_split.h"
#include "launchers.h"

// Scratch of xdit_attn_fwd_noalloc: the balanced launch's partial results and range counter live
// here instead of in a caller workspace.  One copy per GPU the library runs on, held until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress; the
// device address it yields (per device) is what the launches receive.
static __device__ __align__(256) unsigned char scratch[XDIT_ATTN_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int elem_size(int dtype) {
  switch (dtype) {
    case XDIT_DTYPE_BF16:
    case XDIT_DTYPE_FP16: return 2;
    case XDIT_DTYPE_FP32: return 4;
    case XDIT_DTYPE_FP8_E4M3FN: return 1;
    default: return 0;
  }
}

// Every row of a tensor must start on a 16-byte boundary: base aligned, strides multiples of
// 16 bytes.  The S stride must stay below 2^24 bytes: tile loads address a row as "64-bit uniform
// base + 32-bit per-lane offset" and form the offset with a 24-bit multiply (row < 64).
int check_tensor(const char* name, const void* p, const xdit_strides& st, int esize, int D) {
  if (p == nullptr) return fail(XDIT_ERR_INVALID_ARG, "%s is NULL", name);
  if (!aligned16(p)) return fail(XDIT_ERR_INVALID_ARG, "%s is not 16-byte aligned", name);
  const int64_t m = 16 / esize;
  if (st.b % m || st.h % m || st.s % m)
    return fail(XDIT_ERR_INVALID_ARG, "%s: strides (%lld,%lld,%lld) must be multiples of %lld elements",
                name, (long long)st.b, (long long)st.h, (long long)st.s, (long long)m);
  if (st.s < D) return fail(XDIT_ERR_INVALID_ARG, "%s: S stride %lld is smaller than head_dim %d", name, (long long)st.s, D);
  if (st.b < 0 || st.h < 0) return fail(XDIT_ERR_INVALID_ARG, "%s: negative stride", name);
  if (st.s * esize >= (int64_t(1) << 24))
    return fail(XDIT_ERR_INVALID_ARG, "%s: S stride of %lld bytes is too large", name, (long long)(st.s * esize));
  return 0;
}

// head_dim the 16-bit MFMA kernel is built for that holds a tensor head_dim of D (64 or 128; the
// kernel treats the columns the tensors do not have as zeros), 0 if there is none.
int kernel_head_dim(int D) { return D <= 0 || D % 8 != 0 || D > 128 ? 0 : (D <= 64 ? 64 : 128); }

bool mfma16_path(const xdit_attn_args* a) {
  return (a->dtype == XDIT_DTYPE_BF16 || a->dtype == XDIT_DTYPE_FP16) && kernel_head_dim(a->D) != 0;
}

// How the 16-bit and fp8 kernels are launched: query rows per workgroup (384, 256 or 128, i.e. 12,
// 8 or 4 wavefronts sharing each K/V tile) and whether the last round of query tiles is balanced
// over the compute units.  Of the up to six options the one with the shortest estimated time:
//   time = rate * (KV iterations of the busiest workgroup) * rows * (workgroups sharing its compute unit)
//          + (segments of that workgroup) * (workgroups sharing ...) * (exposed cost of a segment's prologue and epilogue)
//          + for a balanced launch: its extra launches, and the partial results a compute unit writes and folds.
// `plain`: the launch will not be balanced (a call without a workspace); `fold_only`: the ring step,
// whose shared tiles are folded inside the attention kernel (plans of at most 16 parts per tile and
// 128- or 256-row workgroups, and about 25 us for the fold on top).  fp8 at head_dim 64 is planned
// with the fp8 constants of head_dim 128.
// Rate and segment cost depend on what a compute unit holds.  One 4-wavefront workgroup leaves
// every SIMD a single wavefront with nothing to overlap its softmax with (1.5 times the time per
// row of 12 wavefronts); two of them hide each other's prologue and epilogue, which a lone 8- or
// 12-wavefront workgroup exposes in full (what decides cross-attention on a few dozen keys).
// Balancing pays wherever the tiles leave compute units idle in the last round (the best plain
// launch is 21 % slower on average than the best of the six, up to 3.8 times on a few heads of
// 1000 to 3000 tokens) and costs a few per cent where they do not.  The constants (ns per query
// row and KV tile; us) are fitted to the times of every option, taken at settled clocks, on 413
// 16-bit problems (B*H 1..48, S 1024..118800, head_dim 64..128; self-attention, ring chunks and
// cross-attention on 77..4608 keys) and 207 fp8 problems.  There the choice is 1.0 % (head_dim
// 128), 1.4 % (64) and 0.6 % (fp8) slower than the fastest option on average, 11 % at worst; on
// 140 problems kept out of an earlier fit of the same form, 1.4 % and 2.0 %.
struct LaunchChoice {
  int rows;    // query rows per workgroup
  int policy;  // AttnParams::split_policy: 1 plain launch, 2 balanced when the planner offers a plan
};

LaunchChoice choose_launch(const xdit_attn_args* a, bool plain = false, bool fold_only = false) {
  LaunchChoice best = {128, 1};
  const int D = kernel_head_dim(a->D);
  if (D == 0) return best;
  const bool fp8 = a->dtype == XDIT_DTYPE_FP8_E4M3FN;
  const int cus = xdit::resident_cus(a->cu_count);
  const int64_t bh = (int64_t)a->B * a->H;
  const int64_t nt = (a->Sk + xdit::kKeysPerTile - 1) / xdit::kKeysPerTile + (a->Sk2 + xdit::kKeysPerTile - 1) / xdit::kKeysPerTile;
  static const int kRows[3] = {384, 256, 128};
  // 16-bit: {384 rows, 256 rows, 128 rows with two workgroups on the compute unit, 128 rows alone}
  static const double kRate128[4] = {5.65, 5.88, 6.93, 8.65}, kRate64[4] = {3.59, 3.56, 4.26, 6.17};
  static const double kSeg128[4] = {8.25, 6.36, 2.05, 6.57}, kSeg64[4] = {2.57, 1.70, 0.42, 2.18};
  const double* rate = D == 64 ? kRate64 : kRate128;
  const double* seg_us = D == 64 ? kSeg64 : kSeg128;
  // a balanced launch: its extra launches, and the partial results per compute unit (us per thousand rows)
  const double split_us = D == 64 ? 1.73 : 3.72;
  const double parts_us = D == 64 ? 18.12 : 28.82;
  // fp8 (head_dim 128, up to three 4-wavefront workgroups per compute unit):
  // {384 rows, 256 rows, 128 rows x 3 / x 2 / alone}
  static const double kRateFp8[5] = {3.64, 4.01, 4.02, 4.99, 6.06}, kSegFp8[5] = {6.18, 5.00, 0.16, 1.62, 5.70};
  const double split_fp8_us = 1.04, parts_fp8_us = 30.50;
  double best_cost = -1;
  for (int i = 0; i < 3; i++) {
    const int rows = kRows[i];
    if (a->rows_per_workgroup != 0 && a->rows_per_workgroup != rows) continue;  // validated by check_tuning
    const int per_cu = rows == 128 ? (fp8 ? 3 : 2) : 1;  // workgroups resident per compute unit
    const int64_t tiles = bh * ((a->Sq + rows - 1) / rows);
    if (tiles > 0x7fffffff) continue;
    const int slots = cus * per_cu;
    for (int policy = 1; policy <= 2; policy++) {
      if ((plain || a->balance == 1) && policy == 2) continue;
      xdit::AttnParams q;
      std::memset(&q, 0, sizeof(q));
      q.Sk = (int)a->Sk; q.Sk2 = (int)a->Sk2; q.total_tiles = (int)tiles;
      q.streamed_ok = a->streamed_sharing != 0;
      q.split_policy = policy;
      if (policy == 2) {
        xdit::plan_split(q, rows, slots, D, 2, fp8 ? 1 : xdit::kClaimsPerWorkgroup, !fp8, fold_only);
        if (q.split_units == 0) continue;  // no balanced plan for this shape
      } else if (a->balance == 2 && !plain) {
        // a balanced plan is to be taken when there is one: the plain launch only stands in without
        xdit::AttnParams t = q;
        t.split_policy = 2;
        xdit::plan_split(t, rows, slots, D, 2, fp8 ? 1 : xdit::kClaimsPerWorkgroup, !fp8, fold_only);
        if (t.split_units != 0) continue;
      }
      int64_t sharing = (tiles + cus - 1) / cus;  // workgroups on the busiest compute unit at once
      if (sharing > per_cu || q.split_units) sharing = per_cu;
      // rounds of resident workgroups; a long plain launch streams its workgroups through the slots
      const double rounds = q.split_units ? (double)(q.split_full / slots)
                            : tiles <= 4 * (int64_t)slots ? (double)((tiles + slots - 1) / slots) : (double)tiles / slots + 0.5;
      const double units = rounds * nt + (q.split_units ? q.split_share : 0);
      const double segs = rounds + (q.split_units ? 1 : 0);
      // partial results written and folded, in thousands of rows per compute unit
      const double parts = q.split_units ? (double)(tiles - q.split_full) * q.split_pmax * rows / cus * 1e-3 : 0.0;
      double cost;
      // the ring step folds its shared tiles inside the attention kernel: a slice per workgroup at its end, or the whole
      // tile by whoever completes it, one round trip to memory after the other (measured: about 25 us)
      const double fold_us = fold_only && q.split_units ? 25.0 : 0.0;
      if (fp8) {
        const int cls = rows == 128 ? 5 - (int)sharing : i;
        cost = kRateFp8[cls] * units * rows * (double)sharing * 1e-3 + kSegFp8[cls] * segs * (double)sharing + (q.split_units ? split_fp8_us + parts_fp8_us * parts : 0.0) + fold_us;
      } else {
        const int cls = rows == 128 ? (sharing > 1 ? 2 : 3) : i;
        cost = rate[cls] * units * rows * (double)sharing * 1e-3 + seg_us[cls] * segs * (double)sharing + (q.split_units ? split_us + parts_us * parts : 0.0) + fold_us;
      }
      if (best_cost < 0 || cost < best_cost) { best.rows = rows; best.policy = policy; best_cost = cost; }
    }
  }
  return best;
}

// The two tuning fields of xdit_attn_args.
int check_tuning(const xdit_attn_args* a) {
  const int r = a->rows_per_workgroup;
  if (r != 0 && r != 128 && r != 256 && r != 384)
    return fail(XDIT_ERR_INVALID_ARG, "rows_per_workgroup %d must be 0, 128, 256 or 384", r);
  if (a->cu_count < 0 || a->cu_count > 4096) return fail(XDIT_ERR_INVALID_ARG, "cu_count %d must be between 0 and 4096", a->cu_count);
  if (a->balance < 0 || a->balance > 2) return fail(XDIT_ERR_INVALID_ARG, "balance %d must be 0, 1 or 2", a->balance);
  if (a->reserved0 != 0) return fail(XDIT_ERR_INVALID_ARG, "reserved0 must be 0");
  return 0;
}

// Validates one prologue job and fills the kernel parameters.
int fill_prologue(const xdit_prologue_args* a, xdit::PrologueParams& p) {
  if (a->struct_size != sizeof(xdit_prologue_args))
    return fail(XDIT_ERR_INVALID_ARG, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(xdit_prologue_args));
  if (a->dtype != XDIT_DTYPE_BF16 && a->dtype != XDIT_DTYPE_FP16 && a->dtype != XDIT_DTYPE_FP32)
    return fail(XDIT_ERR_INVALID_ARG, "dtype %d must be bf16, fp16 or fp32", a->dtype);
  if (a->B <= 0 || a->H <= 0 || a->S <= 0) return fail(XDIT_ERR_INVALID_ARG, "B, H, S must be positive");
  if (a->S > (int64_t(1) << 30) || (int64_t)a->B * a->H * a->S > (int64_t(1) << 40))
    return fail(XDIT_ERR_INVALID_ARG, "tensor too large for one launch");
  if (a->D <= 0 || a->D % 8 != 0 || a->D > 512) return fail(XDIT_ERR_UNSUPPORTED, "head_dim %d: need a multiple of 8, at most 512", a->D);
  if (a->norm < XDIT_NORM_NONE || a->norm > XDIT_NORM_TOKEN) return fail(XDIT_ERR_INVALID_ARG, "unknown norm mode %d", a->norm);
  if (a->rope < XDIT_ROPE_NONE || a->rope > XDIT_ROPE_WAN) return fail(XDIT_ERR_INVALID_ARG, "unknown rope mode %d", a->rope);
  if (a->norm != XDIT_NORM_NONE && !(a->eps >= 0.f && std::isfinite(a->eps))) return fail(XDIT_ERR_INVALID_ARG, "eps must be finite and >= 0");
  const int es = elem_size(a->dtype);
  int rc;
  if ((rc = check_tensor("x", a->x, a->x_stride, es, a->D))) return rc;
  if ((rc = check_tensor("y", a->y, a->y_stride, es, a->D))) return rc;
  if (a->weight != nullptr && !aligned16(a->weight)) return fail(XDIT_ERR_INVALID_ARG, "weight is not 16-byte aligned");
  const int cpr = a->D / 8;
  const bool cpr_pow2 = (cpr & (cpr - 1)) == 0;
  if (a->norm == XDIT_NORM_TOKEN) {
    if (!cpr_pow2 || cpr > 64) return fail(XDIT_ERR_UNSUPPORTED, "token-wide norm needs head_dim/8 to be a power of two <= 64 (head_dim %d)", a->D);
    if ((int64_t)a->H * a->D > xdit::prologue_max_token_elems())
      return fail(XDIT_ERR_UNSUPPORTED, "token-wide norm supports H*D <= %d (got %lld)", xdit::prologue_max_token_elems(), (long long)a->H * a->D);
  }
  if (a->rope != XDIT_ROPE_NONE) {
    if (a->cos == nullptr || a->sin == nullptr) return fail(XDIT_ERR_INVALID_ARG, "cos / sin are NULL");
    if (!aligned16(a->cos) || !aligned16(a->sin) || a->rope_stride % 4 != 0 || a->rope_stride < 0)
      return fail(XDIT_ERR_INVALID_ARG, "cos / sin must be 16-byte aligned with a row stride that is a non-negative multiple of 4");
    if (a->rope_row0 < 0 || a->rope_rows < 0 || a->rope_row0 + a->rope_rows > a->S)
      return fail(XDIT_ERR_INVALID_ARG, "rope rows [%lld, %lld) do not lie within S=%lld", (long long)a->rope_row0, (long long)(a->rope_row0 + a->rope_rows), (long long)a->S);
    if (a->rope == XDIT_ROPE_SPLIT_HALF && (!cpr_pow2 || cpr < 2 || cpr > 64))
      return fail(XDIT_ERR_UNSUPPORTED, "split-half rotation needs head_dim/8 to be a power of two in [2, 64] (head_dim %d)", a->D);
  }
  std::memset(&p, 0, sizeof(p));
  p.x = a->x; p.y = a->y; p.weight = a->norm != XDIT_NORM_NONE ? a->weight : nullptr;
  p.cos = a->cos; p.sin = a->sin;
  p.xs_b = a->x_stride.b; p.xs_h = a->x_stride.h; p.xs_s = a->x_stride.s;
  p.ys_b = a->y_stride.b; p.ys_h = a->y_stride.h; p.ys_s = a->y_stride.s;
  p.rope_stride = a->rope_stride;
  p.B = a->B; p.H = a->H; p.S = (int)a->S; p.D = a->D;
  p.rows = (int64_t)a->B * a->S * a->H;
  p.norm = a->norm; p.rope_mode = a->rope;
  p.rope_row0 = (int)a->rope_row0; p.rope_rows = (int)a->rope_rows;
  int lpr = 1;
  while (lpr < cpr) lpr <<= 1;
  p.lpr = lpr;
  if ((p.rows * lpr + 255) / 256 > 0x7fffffffLL) return fail(XDIT_ERR_INVALID_ARG, "tensor too large for one launch");
  p.eps = a->eps;
  p.inv_n = 1.0f / (float)(a->norm == XDIT_NORM_TOKEN ? (int64_t)a->H * a->D : (int64_t)a->D);
  return 0;
}

}  // namespace

extern "C" {

const char* xdit_attn_last_error(void) { return g_err; }

int xdit_attn_abi_version(void) { return XDIT_ATTN_ABI_VERSION; }

static int attn_fwd_impl(const xdit_attn_args* a, const xdit_ring_acc* acc) {
  g_err[0] = 0;
  if (a == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  if (a->struct_size != sizeof(xdit_attn_args))
    return fail(XDIT_ERR_INVALID_ARG, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(xdit_attn_args));
  const int es = elem_size(a->dtype);
  if (es == 0) return fail(XDIT_ERR_INVALID_ARG, "unknown dtype %d", a->dtype);
  if (a->causal != 0) return fail(XDIT_ERR_UNSUPPORTED, "causal attention is not implemented (DiT attention is non-causal)");
  if (a->B <= 0 || a->H <= 0) return fail(XDIT_ERR_INVALID_ARG, "B=%d H=%d must be positive", a->B, a->H);
  if (a->Sq <= 0 || a->Sk <= 0 || a->Sk2 < 0)
    return fail(XDIT_ERR_INVALID_ARG, "Sq=%lld Sk=%lld Sk2=%lld: need Sq>0, Sk>0, Sk2>=0", (long long)a->Sq, (long long)a->Sk, (long long)a->Sk2);
  if (a->Sq > (int64_t(1) << 30) || a->Sk > (int64_t(1) << 30) || a->Sk2 > (int64_t(1) << 30))
    return fail(XDIT_ERR_INVALID_ARG, "sequence length above 2^30");
  if ((int64_t)a->B * a->H * ((a->Sq + 31) / 32) > (int64_t(1) << 30))
    return fail(XDIT_ERR_INVALID_ARG, "B*H*Sq too large for one launch");
  if (!(a->softmax_scale > 0.f) || !std::isfinite(a->softmax_scale))
    return fail(XDIT_ERR_INVALID_ARG, "softmax_scale must be finite and > 0");
  if (a->D <= 0 || a->D % 8 != 0 || a->D > 256) return fail(XDIT_ERR_UNSUPPORTED, "head_dim %d: need a multiple of 8, at most 256", a->D);

  if (int rc0 = check_tuning(a)) return rc0;

  int out_dtype = a->out_dtype;
  if (a->dtype == XDIT_DTYPE_FP8_E4M3FN) {
    if (out_dtype != XDIT_DTYPE_BF16 && out_dtype != XDIT_DTYPE_FP16)
      return fail(XDIT_ERR_INVALID_ARG, "fp8 inputs need a bf16 or fp16 output");
  } else if (out_dtype != a->dtype) {
    return fail(XDIT_ERR_INVALID_ARG, "out_dtype %d must equal dtype %d", out_dtype, a->dtype);
  }
  int rc;
  if ((rc = check_tensor("q", a->q, a->q_stride, es, a->D))) return rc;
  if ((rc = check_tensor("k", a->k, a->k_stride, es, a->D))) return rc;
  if ((rc = check_tensor("v", a->v, a->v_stride, es, a->D))) return rc;
  if (a->Sk2 > 0) {
    if ((rc = check_tensor("k2", a->k2, a->k2_stride, es, a->D))) return rc;
    if ((rc = check_tensor("v2", a->v2, a->v2_stride, es, a->D))) return rc;
  }
  if (acc == nullptr || a->out != nullptr)
    if ((rc = check_tensor("out", a->out, a->out_stride, elem_size(out_dtype), a->D))) return rc;
  if (acc != nullptr) {
    if (acc->struct_size != sizeof(xdit_ring_acc))
      return fail(XDIT_ERR_INVALID_ARG, "acc struct_size %u != %zu (ABI mismatch)", acc->struct_size, sizeof(xdit_ring_acc));
    if (a->dtype == XDIT_DTYPE_FP8_E4M3FN ? (a->D != 128 && a->D != 64) : a->D > 128)
      return fail(XDIT_ERR_UNSUPPORTED, "the fused ring step needs head_dim at most 128 (fp8: 128 or 64), got %d", a->D);
    if ((rc = check_tensor("acc_out", acc->acc_out, acc->acc_out_stride, 4, a->D))) return rc;
    if (acc->acc_lse == nullptr) return fail(XDIT_ERR_INVALID_ARG, "acc_lse is NULL");
    if (acc->acc_lse_stride.b < 0 || acc->acc_lse_stride.h < 0 || acc->acc_lse_stride.s <= 0)
      return fail(XDIT_ERR_INVALID_ARG, "acc_lse strides must be non-negative (row stride positive)");
    if (acc->discard_acc_out != 0 && a->out == nullptr)
      return fail(XDIT_ERR_INVALID_ARG, "discard_acc_out needs args->out to receive the result");
  }
  if (a->lse != nullptr && (a->lse_stride_b < 0 || a->lse_stride_h < a->Sq))
    return fail(XDIT_ERR_INVALID_ARG, "lse strides (%lld,%lld) do not hold Sq=%lld rows", (long long)a->lse_stride_b, (long long)a->lse_stride_h, (long long)a->Sq);

  xdit::AttnParams p;
  std::memset(&p, 0, sizeof(p));
  p.q = a->q; p.k = a->k; p.v = a->v; p.k2 = a->k2; p.v2 = a->v2; p.out = a->out; p.lse = a->lse;
  p.qs_b = a->q_stride.b; p.qs_h = a->q_stride.h; p.qs_s = a->q_stride.s;
  p.ks_b = a->k_stride.b; p.ks_h = a->k_stride.h; p.ks_s = a->k_stride.s;
  p.vs_b = a->v_stride.b; p.vs_h = a->v_stride.h; p.vs_s = a->v_stride.s;
  p.k2s_b = a->k2_stride.b; p.k2s_h = a->k2_stride.h; p.k2s_s = a->k2_stride.s;
  p.v2s_b = a->v2_stride.b; p.v2s_h = a->v2_stride.h; p.v2s_s = a->v2_stride.s;
  p.os_b = a->out_stride.b; p.os_h = a->out_stride.h; p.os_s = a->out_stride.s;
  p.ls_b = a->lse_stride_b; p.ls_h = a->lse_stride_h;
  p.q_descale = a->q_descale; p.k_descale = a->k_descale; p.v_descale = a->v_descale;
  p.ds_b = a->descale_stride_b; p.ds_h = a->descale_stride_h;
  p.B = a->B; p.H = a->H;
  p.Sq = (int)a->Sq; p.Sk = (int)a->Sk; p.Sk2 = (int)a->Sk2;
  p.scale = a->softmax_scale;
  p.cu_count = a->cu_count;
  p.streamed_ok = a->streamed_sharing != 0;
  if (acc != nullptr) {
    p.acc_out = acc->acc_out; p.acc_lse = acc->acc_lse;
    p.ao_b = acc->acc_out_stride.b; p.ao_h = acc->acc_out_stride.h; p.ao_s = acc->acc_out_stride.s;
    p.al_b = acc->acc_lse_stride.b; p.al_h = acc->acc_lse_stride.h; p.al_s = acc->acc_lse_stride.s;
    p.acc_first = acc->first != 0;
    p.acc_store = acc->discard_acc_out == 0;
  }
  if (a->workspace != nullptr && a->workspace_bytes >= (int64_t)xdit::kCounterRegionBytes && aligned16(a->workspace)) {
    p.ws_out = a->workspace;
    p.ws_preserved = a->workspace_preserved != 0;
    p.ws_bytes = (size_t)a->workspace_bytes;
  }
  hipStream_t stream = (hipStream_t)a->stream;

  const bool fp8 = a->dtype == XDIT_DTYPE_FP8_E4M3FN;
  if (fp8 && a->D != 128 && a->D != 64) return fail(XDIT_ERR_UNSUPPORTED, "fp8 attention supports head_dim 128 and 64 only (got %d)", a->D);
  if (!fp8 && !mfma16_path(a) && a->D > 128) return fail(XDIT_ERR_UNSUPPORTED, "head_dim %d above 128 is not implemented", a->D);
  // A workspace whose contents the caller does not vouch for gets its counters cleared, whatever
  // launch follows: the next call on it may then say "preserved" whether this one is balanced or not.
  if (p.ws_out != nullptr && !p.ws_preserved) xdit::launch_counter_reset(p.ws_out, stream);
  hipError_t e;
  if (fp8 || mfma16_path(a)) {
    const int D = fp8 ? a->D : kernel_head_dim(a->D);
    if (!fp8) p.d_actual = a->D;
    const bool fused = acc != nullptr;
    LaunchChoice c = choose_launch(a, p.ws_out == nullptr, fused);  // no workspace: the shape that suits a plain launch
    p.split_policy = c.policy;
    if (c.policy == 2) {
      // a workspace too small for the chosen balanced plan: the best PLAIN launch, not that shape run plain
      xdit::AttnParams plan;
      const size_t need = fp8 ? xdit::attn_fwd_fp8_workspace(p, D, c.rows, &plan, fused) : xdit::attn_fwd_16_workspace(p, D, c.rows, &plan, fused);
      if (need > p.ws_bytes) {
        c = choose_launch(a, true, fused);
        p.split_policy = c.policy;
      }
    }
    if (fp8) e = xdit::launch_attn_fwd_fp8(p, D, out_dtype == XDIT_DTYPE_FP16, c.rows, stream);
    else e = fused ? xdit::launch_attn_fwd_16_ring(p, a->dtype == XDIT_DTYPE_FP16, D, c.rows, stream)
                   : xdit::launch_attn_fwd_16(p, a->dtype == XDIT_DTYPE_FP16, D, c.rows, stream);
  } else {
    e = xdit::launch_attn_fwd_f32(p, a->D, stream);  // fp32 tensors: every 16-bit case went to the 16-bit kernel
  }
  if (e != hipSuccess) return fail(XDIT_ERR_LAUNCH, "attention launch failed: %s", hipGetErrorString(e));
  return XDIT_OK;
}

int xdit_attn_fwd(const xdit_attn_args* a) { return attn_fwd_impl(a, nullptr); }

int xdit_attn_fwd_noalloc(const xdit_attn_args* a) {
  g_err[0] = 0;
  if (a == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  const int64_t need = xdit_attn_workspace_bytes(a);  // validates struct_size, shape and tuning fields
  if (need < 0) return (int)need;
  if (need > (int64_t)XDIT_ATTN_NOALLOC_SCRATCH_BYTES)
    return fail(XDIT_ERR_INVALID_ARG,
                "this problem needs %lld bytes of scratch, xdit_attn_fwd_noalloc holds %lld: call xdit_attn_fwd with a workspace of the caller, or set balance = 1 (plain launch, no scratch)",
                (long long)need, (long long)XDIT_ATTN_NOALLOC_SCRATCH_BYTES);
  xdit_attn_args b = *a;
  b.workspace = nullptr;
  b.workspace_bytes = 0;
  b.workspace_preserved = 0;
  if (need > 0) {
    // device address of this GPU's copy of the array, looked up once per device with that device current
    static std::atomic<void*> scratch_ptr[xdit::kMaxDevices];
    const int slot = xdit::current_device_slot();
    void* ptr = scratch_ptr[slot].load(std::memory_order_acquire);
    if (ptr == nullptr) {
      const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
      if (e != hipSuccess || ptr == nullptr)
        return fail(XDIT_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
      scratch_ptr[slot].store(ptr, std::memory_order_release);
    }
    b.workspace = ptr;
    b.workspace_bytes = (int64_t)XDIT_ATTN_NOALLOC_SCRATCH_BYTES;
    // The array starts out zeroed and only this library writes it, so its counters are as the last
    // call left them: at zero, unless that call failed part-way (then a kernel clears them first).
    static std::atomic<int> scratch_dirty[xdit::kMaxDevices];
    b.workspace_preserved = scratch_dirty[slot].load(std::memory_order_relaxed) == 0;
    const int rc = attn_fwd_impl(&b, nullptr);
    scratch_dirty[slot].store(rc != XDIT_OK, std::memory_order_relaxed);
    return rc;
  }
  return attn_fwd_impl(&b, nullptr);
}

int xdit_attn_fwd_accumulate(const xdit_attn_args* a, const xdit_ring_acc* acc) {
  if (acc == nullptr) {
    g_err[0] = 0;
    return fail(XDIT_ERR_INVALID_ARG, "acc is NULL");
  }
  return attn_fwd_impl(a, acc);
}

int64_t xdit_attn_workspace_bytes(const xdit_attn_args* a) {
  g_err[0] = 0;
  if (a == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  if (a->struct_size != sizeof(xdit_attn_args))
    return fail(XDIT_ERR_INVALID_ARG, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(xdit_attn_args));
  if (a->B <= 0 || a->H <= 0 || a->Sq <= 0 || a->Sk <= 0 || a->Sk2 < 0 || a->Sq > (int64_t(1) << 30) ||
      a->Sk > (int64_t(1) << 30) || a->Sk2 > (int64_t(1) << 30) ||
      (int64_t)a->B * a->H * ((a->Sq + 31) / 32) > (int64_t(1) << 30))
    return fail(XDIT_ERR_INVALID_ARG, "bad shape");
  if (int rc0 = check_tuning(a)) return rc0;
  xdit::AttnParams p;
  std::memset(&p, 0, sizeof(p));
  p.B = a->B; p.H = a->H; p.Sq = (int)a->Sq; p.Sk = (int)a->Sk; p.Sk2 = (int)a->Sk2;
  p.cu_count = a->cu_count;
  p.streamed_ok = a->streamed_sharing != 0;
  if (!(a->dtype == XDIT_DTYPE_FP8_E4M3FN && (a->D == 128 || a->D == 64)) && !mfma16_path(a)) return 0;
  const LaunchChoice c = choose_launch(a);
  p.split_policy = c.policy;
  if (a->dtype == XDIT_DTYPE_FP8_E4M3FN) return (int64_t)xdit::attn_fwd_fp8_workspace(p, a->D, c.rows);
  return (int64_t)xdit::attn_fwd_16_workspace(p, kernel_head_dim(a->D), c.rows);
}

int xdit_attn_launch_plan(const xdit_attn_args* a, xdit_launch_plan* out) {
  g_err[0] = 0;
  if (a == nullptr || out == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args or plan is NULL");
  if (a->struct_size != sizeof(xdit_attn_args))
    return fail(XDIT_ERR_INVALID_ARG, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(xdit_attn_args));
  if (out->struct_size != sizeof(xdit_launch_plan))
    return fail(XDIT_ERR_INVALID_ARG, "plan struct_size %u != %zu (ABI mismatch)", out->struct_size, sizeof(xdit_launch_plan));
  if (a->B <= 0 || a->H <= 0 || a->Sq <= 0 || a->Sk <= 0 || a->Sk2 < 0 || a->Sq > (int64_t(1) << 30) ||
      a->Sk > (int64_t(1) << 30) || a->Sk2 > (int64_t(1) << 30) ||
      (int64_t)a->B * a->H * ((a->Sq + 31) / 32) > (int64_t(1) << 30))
    return fail(XDIT_ERR_INVALID_ARG, "bad shape");
  if (int rc0 = check_tuning(a)) return rc0;
  const bool fp8 = a->dtype == XDIT_DTYPE_FP8_E4M3FN && (a->D == 128 || a->D == 64);
  const bool b16 = mfma16_path(a);
  xdit::AttnParams p, q;
  std::memset(&p, 0, sizeof(p));
  p.B = a->B; p.H = a->H; p.Sq = (int)a->Sq; p.Sk = (int)a->Sk; p.Sk2 = (int)a->Sk2;
  p.cu_count = a->cu_count;
  p.streamed_ok = a->streamed_sharing != 0;
  if (a->dtype == XDIT_DTYPE_FP32 && a->D > 0 && a->D % 8 == 0 && a->D <= 128) {
    // the fp32 kernel: one workgroup per query tile, no shared last round, no workspace
    const int rows = xdit::attn_fwd_f32_rows(p);
    const int keys = rows == 64 ? 64 : 32;
    const uint32_t size = out->struct_size;
    std::memset(out, 0, sizeof(*out));
    out->struct_size = size;
    out->rows_per_workgroup = rows;
    out->query_tiles = (int32_t)(a->B * a->H * ((a->Sq + rows - 1) / rows));
    out->kv_iterations = (int32_t)((a->Sk + keys - 1) / keys + (a->Sk2 + keys - 1) / keys);
    out->whole_tiles = out->query_tiles;
    out->workgroups = (out->query_tiles + 7) / 8 * 8;
    return XDIT_OK;
  }
  if (!fp8 && !b16) return fail(XDIT_ERR_UNSUPPORTED, "no launch plan for this dtype / head_dim");
  const bool ring_step = out->ring_step != 0;
  const LaunchChoice choice = choose_launch(a, false, ring_step);
  const int rows = choice.rows;
  p.split_policy = choice.policy;
  const size_t need = fp8 ? xdit::attn_fwd_fp8_workspace(p, a->D, rows, &q, ring_step) : xdit::attn_fwd_16_workspace(p, kernel_head_dim(a->D), rows, &q, ring_step);
  const uint32_t size = out->struct_size;
  std::memset(out, 0, sizeof(*out));
  out->struct_size = size;
  out->ring_step = ring_step;
  out->rows_per_workgroup = rows;
  out->query_tiles = q.total_tiles;
  out->kv_iterations = (int32_t)((a->Sk + xdit::kKeysPerTile - 1) / xdit::kKeysPerTile + (a->Sk2 + xdit::kKeysPerTile - 1) / xdit::kKeysPerTile);
  out->workspace_bytes = (int64_t)need;
  out->whole_tiles = q.split_units ? q.split_full : q.total_tiles;
  out->ranges = q.split_units;
  out->range_len = q.split_len;
  out->slots_per_tile = q.split_pmax;
  out->claimers = q.split_claimers;
  out->first_claimer = q.split_units ? (q.split_fuse0 <= q.split_full ? q.split_fuse0 : q.split_full) : 0;
  out->counter = xdit::split_counters(q) > 0 ? 1 : 0;
  out->streamed = q.split_dyn;
  out->fold_in_kernel = q.split_fold;
  out->parts_first = q.split_order;
  if (q.split_dyn) out->range_len = q.split_s0;
  out->workgroups = (int32_t)xdit::split_grid(q);
  return XDIT_OK;
}

int xdit_lse_merge(const xdit_merge_args* a) {
  g_err[0] = 0;
  if (a == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  if (a->struct_size != sizeof(xdit_merge_args))
    return fail(XDIT_ERR_INVALID_ARG, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(xdit_merge_args));
  if (a->block_dtype != XDIT_DTYPE_BF16 && a->block_dtype != XDIT_DTYPE_FP16 && a->block_dtype != XDIT_DTYPE_FP32)
    return fail(XDIT_ERR_INVALID_ARG, "block_dtype %d must be bf16, fp16 or fp32", a->block_dtype);
  if (a->B <= 0 || a->H <= 0 || a->S <= 0) return fail(XDIT_ERR_INVALID_ARG, "B, H, S must be positive");
  if (a->D <= 0 || a->D % 8 != 0 || a->D > 512) return fail(XDIT_ERR_INVALID_ARG, "head_dim %d must be a positive multiple of 8, at most 512", a->D);
  if (a->S > (int64_t(1) << 30)) return fail(XDIT_ERR_INVALID_ARG, "S above 2^30");
  if (a->acc_lse == nullptr || a->block_lse == nullptr) return fail(XDIT_ERR_INVALID_ARG, "acc_lse / block_lse is NULL");
  int rc;
  xdit_strides big = a->acc_out_stride;
  if ((rc = check_tensor("acc_out", a->acc_out, big, 4, a->D))) return rc;
  if ((rc = check_tensor("block_out", a->block_out, a->block_out_stride, elem_size(a->block_dtype), a->D))) return rc;
  if (a->final_out != nullptr) {
    if (a->final_dtype != XDIT_DTYPE_BF16 && a->final_dtype != XDIT_DTYPE_FP16 && a->final_dtype != XDIT_DTYPE_FP32)
      return fail(XDIT_ERR_INVALID_ARG, "final_dtype %d must be bf16, fp16 or fp32", a->final_dtype);
    if ((rc = check_tensor("final_out", a->final_out, a->final_out_stride, elem_size(a->final_dtype), a->D))) return rc;
  }
  xdit::MergeParams p;
  std::memset(&p, 0, sizeof(p));
  p.acc_out = a->acc_out; p.acc_lse = a->acc_lse; p.block_out = a->block_out; p.block_lse = a->block_lse;
  p.final_out = a->final_out;
  p.ao_b = a->acc_out_stride.b; p.ao_h = a->acc_out_stride.h; p.ao_s = a->acc_out_stride.s;
  p.bo_b = a->block_out_stride.b; p.bo_h = a->block_out_stride.h; p.bo_s = a->block_out_stride.s;
  p.fo_b = a->final_out_stride.b; p.fo_h = a->final_out_stride.h; p.fo_s = a->final_out_stride.s;
  p.al_b = a->acc_lse_stride.b; p.al_h = a->acc_lse_stride.h; p.al_s = a->acc_lse_stride.s;
  p.bl_b = a->block_lse_stride.b; p.bl_h = a->block_lse_stride.h; p.bl_s = a->block_lse_stride.s;
  p.B = a->B; p.H = a->H; p.S = (int)a->S; p.D = a->D;
  p.first = a->first;
  p.rows = (int64_t)a->B * a->H * a->S;
  if (p.rows * (a->D / 8) > (int64_t(1) << 38)) return fail(XDIT_ERR_INVALID_ARG, "tensor too large for one launch");
  hipError_t e = xdit::launch_lse_merge(p, a->block_dtype, a->final_dtype, (hipStream_t)a->stream);
  if (e != hipSuccess) return fail(XDIT_ERR_LAUNCH, "merge launch failed: %s", hipGetErrorString(e));
  return XDIT_OK;
}

int xdit_fp8_quant(const xdit_quant_args* a) {
  g_err[0] = 0;
  if (a == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  if (a->struct_size != sizeof(xdit_quant_args))
    return fail(XDIT_ERR_INVALID_ARG, "struct_size %u != %zu (ABI mismatch)", a->struct_size, sizeof(xdit_quant_args));
  if (a->in_dtype != XDIT_DTYPE_BF16 && a->in_dtype != XDIT_DTYPE_FP16 && a->in_dtype != XDIT_DTYPE_FP32)
    return fail(XDIT_ERR_INVALID_ARG, "in_dtype %d must be bf16, fp16 or fp32", a->in_dtype);
  if (a->B <= 0 || a->H <= 0 || a->S <= 0) return fail(XDIT_ERR_INVALID_ARG, "B, H, S must be positive");
  if (a->B * (int64_t)a->H > 65535) return fail(XDIT_ERR_INVALID_ARG, "B*H above 65535");
  if (a->per_tensor && a->B * (int64_t)a->H > 1024) return fail(XDIT_ERR_INVALID_ARG, "per_tensor mode supports B*H <= 1024");
  if (a->D <= 0 || a->D % 8 != 0 || a->D > 2048) return fail(XDIT_ERR_INVALID_ARG, "head_dim %d must be a positive multiple of 8, at most 2048", a->D);
  if (a->S > (int64_t(1) << 30)) return fail(XDIT_ERR_INVALID_ARG, "S above 2^30");
  if (a->descale == nullptr) return fail(XDIT_ERR_INVALID_ARG, "descale is NULL");
  int rc;
  if ((rc = check_tensor("x", a->x, a->x_stride, elem_size(a->in_dtype), a->D))) return rc;
  if (a->y == nullptr) return fail(XDIT_ERR_INVALID_ARG, "y is NULL");
  if ((reinterpret_cast<uintptr_t>(a->y) & 7u) || a->y_stride.b % 8 || a->y_stride.h % 8 || a->y_stride.s % 8)
    return fail(XDIT_ERR_INVALID_ARG, "y must be 8-byte aligned with strides that are multiples of 8");
  if (a->y_stride.s < a->D) return fail(XDIT_ERR_INVALID_ARG, "y: S stride smaller than head_dim");
  if (a->S2 < 0 || a->S2 > (int64_t(1) << 30)) return fail(XDIT_ERR_INVALID_ARG, "S2 must be between 0 and 2^30");
  if (a->S2 > 0) {
    if ((rc = check_tensor("x2", a->x2, a->x2_stride, elem_size(a->in_dtype), a->D))) return rc;
    if (a->y2 == nullptr) return fail(XDIT_ERR_INVALID_ARG, "y2 is NULL");
    if ((reinterpret_cast<uintptr_t>(a->y2) & 7u) || a->y2_stride.b % 8 || a->y2_stride.h % 8 || a->y2_stride.s % 8)
      return fail(XDIT_ERR_INVALID_ARG, "y2 must be 8-byte aligned with strides that are multiples of 8");
    if (a->y2_stride.s < a->D) return fail(XDIT_ERR_INVALID_ARG, "y2: S stride smaller than head_dim");
  }
  const int hb = a->hadamard_block;
  if (hb < 0 || hb > 128 || (hb & (hb - 1)) != 0 || (hb > 1 && a->D % hb != 0))
    return fail(XDIT_ERR_INVALID_ARG, "hadamard_block %d must be 0 or a power of two <= 128 that divides head_dim %d", hb, a->D);
  xdit::QuantParams p;
  std::memset(&p, 0, sizeof(p));
  p.had_block = hb > 1 ? hb : 0;
  p.had_scale = hb > 1 ? 1.0f / std::sqrt((float)hb) : 1.0f;
  p.x = a->x; p.y = a->y; p.amax = a->descale; p.descale = a->descale; p.scale_in = a->scale_in;
  p.xs_b = a->x_stride.b; p.xs_h = a->x_stride.h; p.xs_s = a->x_stride.s;
  p.ys_b = a->y_stride.b; p.ys_h = a->y_stride.h; p.ys_s = a->y_stride.s;
  p.B = a->B; p.H = a->H; p.S = (int)a->S; p.D = a->D;
  p.per_tensor = a->per_tensor ? 1 : 0;
  if (a->S2 > 0) {
    p.x2 = a->x2; p.y2 = a->y2; p.S2 = (int)a->S2;
    p.x2s_b = a->x2_stride.b; p.x2s_h = a->x2_stride.h; p.x2s_s = a->x2_stride.s;
    p.y2s_b = a->y2_stride.b; p.y2s_h = a->y2_stride.h; p.y2s_s = a->y2_stride.s;
  }
  if (a->scratch != nullptr && (reinterpret_cast<uintptr_t>(a->scratch) & 3u) == 0 &&
      a->scratch_bytes >= XDIT_FP8_QUANT_SCRATCH_BYTES(a->B, a->H)) {
    p.partials = (float*)a->scratch;
    p.partial_slots = a->scratch_bytes / 4;
    if (p.partial_slots > 65536) p.partial_slots = 65536;
    const int64_t bh = (int64_t)a->B * a->H;
    if (p.partial_slots < bh) p.partials = nullptr;
  }
  hipError_t e = xdit::launch_fp8_quant(p, a->in_dtype, (hipStream_t)a->stream);
  if (e != hipSuccess) return fail(XDIT_ERR_LAUNCH, "quantiser launch failed: %s", hipGetErrorString(e));
  return XDIT_OK;
}

int xdit_qk_prologue(const xdit_prologue_args* a) {
  g_err[0] = 0;
  if (a == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  xdit::PrologueParams p;
  int rc;
  if ((rc = fill_prologue(a, p))) return rc;
  hipError_t e = xdit::launch_qk_prologue(p, a->dtype, (hipStream_t)a->stream);
  if (e != hipSuccess) return fail(XDIT_ERR_LAUNCH, "prologue launch failed: %s", hipGetErrorString(e));
  return XDIT_OK;
}

int xdit_qk_prologue_batch(const xdit_prologue_args* jobs, int32_t count) {
  g_err[0] = 0;
  if (jobs == nullptr) return fail(XDIT_ERR_INVALID_ARG, "args is NULL");
  if (count < 1 || count > xdit::kPrologueBatchMax)
    return fail(XDIT_ERR_INVALID_ARG, "count %d must be between 1 and %d", count, xdit::kPrologueBatchMax);
  xdit::PrologueBatch b;
  std::memset(&b, 0, sizeof(b));
  b.n = count;
  for (int i = 0; i < count; i++) {
    int rc;
    if ((rc = fill_prologue(&jobs[i], b.job[i]))) return rc;
    if (jobs[i].dtype != jobs[0].dtype || jobs[i].stream != jobs[0].stream)
      return fail(XDIT_ERR_INVALID_ARG, "job %d: every job of a batch must have the dtype and the stream of job 0", i);
    if (jobs[i].norm == XDIT_NORM_TOKEN)
      return fail(XDIT_ERR_UNSUPPORTED, "job %d: the token-wide norm cannot be batched", i);
  }
  hipError_t e = xdit::launch_qk_prologue_batch(b, jobs[0].dtype, (hipStream_t)jobs[0].stream);
  if (e != hipSuccess) return fail(XDIT_ERR_LAUNCH, "prologue launch failed: %s", hipGetErrorString(e));
  return XDIT_OK;
}

}  // extern "C"
