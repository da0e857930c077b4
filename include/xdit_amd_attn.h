/*
 * xdit_amd_attn.h — C ABI of the MI355X (gfx950) attention hot path.
 *
 * One shared library (libxdit_amd_attn.so) exports the entry points below.  They are what a
 * foreign-function binding (ctypes, cffi, pybind, a C++ torch op) of xDiT's attention path would
 * bind on one GPU.  Every pointer is a DEVICE pointer owned by the caller; the library allocates
 * nothing, keeps nothing after return, never synchronises the device and launches on the stream
 * the caller passes.  All strides are in ELEMENTS of the tensor's own dtype.  The innermost
 * (head_dim) stride of every tensor is 1.
 *
 * Return value: 0 on success, a negative xdit_status otherwise; the message of the last failure
 * on the calling thread is available from xdit_attn_last_error().
 *
 * Reference interfaces replaced (paths relative to the xDiT source tree):
 *   - the `(out, lse)` vendor flash-attention forward reached by the backend registry entries
 *     xfuser/core/distributed/attention_backend.py:504-516 (SDPA_FLASH), :534-548 (SDPA_EFFICIENT),
 *     :774-823 (AITER), :887-918 (FLASH), and by the per-step kernel call of the legacy ring loop
 *     xfuser/core/long_ctx_attention/ring/ring_flash_attn.py:105-134            -> xdit_attn_fwd
 *   - the fp8 forward with per-(batch,head) descales, attention_backend.py:617-642 (FLASH_3_FP8)
 *     and :717-772 (AITER_FP8)                                                   -> xdit_attn_fwd (dtype FP8)
 *   - the ring online-softmax merge `update_out_and_lse` called at
 *     ring_flash_attn.py:138 (+ epilogue :145-148) and torch's `_SDPAMerger._merge_one`
 *     (torch/distributed/tensor/experimental/_context_parallel/_attention.py:181-182)
 *                                                                                -> xdit_lse_merge
 *   - `per_tensor_quant`, attention_backend.py:606-615                           -> xdit_fp8_quant
 */
#ifndef XDIT_AMD_ATTN_H
#define XDIT_AMD_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XDIT_ATTN_ABI_VERSION 8

typedef enum {
  XDIT_OK = 0,
  XDIT_ERR_INVALID_ARG = -1,   /* null pointer, bad shape/stride/alignment, unsupported option */
  XDIT_ERR_UNSUPPORTED = -2,   /* a combination this library does not implement (e.g. causal)  */
  XDIT_ERR_LAUNCH = -3         /* the HIP runtime rejected the launch                          */
} xdit_status;

typedef enum {
  XDIT_DTYPE_BF16 = 0,
  XDIT_DTYPE_FP16 = 1,
  XDIT_DTYPE_FP32 = 2,
  XDIT_DTYPE_FP8_E4M3FN = 3    /* OCP e4m3fn (max 448), the fp8 format of gfx950 */
} xdit_dtype;

/* Logical tensor (B, H, S, D) with arbitrary B/H/S element strides; D stride is 1.
 * BHSD-contiguous:                stride = {H*S*D, S*D, D}
 * BSHD-contiguous viewed as BHSD: stride = {S*H*D, D, H*D}                                   */
typedef struct {
  int64_t b, h, s;
} xdit_strides;

/*
 * Non-causal scaled-dot-product attention forward returning the output and the per-row
 * log-sum-exp (natural log, softmax scale included):
 *     s_ij = softmax_scale * sum_d q_id k_jd ,  j over Sk keys of (k,v) then Sk2 keys of (k2,v2)
 *     out_i = sum_j softmax_j(s_ij) v_j ,  lse_i = log sum_j exp(s_ij)
 * For FP8 inputs q,k,v are multiplied by q_descale[b,h], k_descale[b,h], v_descale[b,h] first.
 * head_dim: a multiple of 8; bf16 / fp16 / fp32 up to 128 (bf16 and fp16 on the 16-bit matrix
 * cores at every such head_dim, at the cost of the next of 64 / 128; fp32 on the fp32 matrix
 * cores), fp8 128 or 64.
 * Replaces: attention_backend.py:504-516/:774-823/:887-918 (+ :617-642, :717-772 for fp8) and the
 * kernel call at ring_flash_attn.py:123-134.  The optional second KV segment replaces the
 * torch.cat of joint (text) keys/values at usp.py:239-241 / ring_flash_attn.py:89-100.
 */
typedef struct {
  uint32_t struct_size;        /* = sizeof(xdit_attn_args) */
  int32_t dtype;               /* xdit_dtype of q, k, v, k2, v2 */
  int32_t out_dtype;           /* xdit_dtype of out: same as dtype for bf16/fp16/fp32; bf16 or fp16 for fp8 */
  int32_t causal;              /* must be 0 */
  int32_t B, H, D;             /* batch, heads (Hq == Hk), head_dim */
  int32_t rows_per_workgroup;  /* 0 = chosen by the library; 128, 256 or 384 = that workgroup shape
                                  (bf16 / fp16 / fp8 kernels; a tuning and testing aid) */
  int64_t Sq, Sk, Sk2;         /* query rows; keys in segment 1; keys in segment 2 (0 = none) */
  float softmax_scale;         /* > 0 */
  int32_t cu_count;            /* 0 = plan the launch for the compute units of the current device;
                                  > 0 = for that many (tuning, testing, capacity planning) */
  int32_t streamed_sharing;    /* 0 (default): the work geometry of a launch is fixed, so results are
                                  reproducible bit for bit from call to call, as those of the vendor
                                  forwards this call replaces are (the reference's `deterministic`
                                  option concerns its backward pass only: ring_flash_attn.py:190, :206,
                                  :229).  != 0 opts in to a balanced launch that hands KV iterations of
                                  a shared query tile to whichever workgroup is free: 1-2 % faster on
                                  some shapes, results then reproducible only to rounding (the last
                                  bit of some outputs) */
  int32_t workspace_preserved; /* != 0: the caller vouches that nothing but this library has written
                                  `workspace` since an earlier call of this library that was given the
                                  same pointer, returned XDIT_OK and had 0 here on the first call after
                                  allocating the buffer (any such call will do: balanced or not, any
                                  dtype; a call that is given a workspace of at least 16 KiB with 0 here
                                  clears the counters at its start with a small launch).  The counters are
                                  then still zero and that launch is spared.  0 is always valid */
  int32_t balance;             /* 0 = the library decides from its time estimate whether a launch given a
                                  workspace is balanced; 1 = never (plain launch); 2 = whenever the planner
                                  offers a balanced plan (a tuning and testing aid, like rows_per_workgroup) */
  int32_t reserved0;           /* must be 0 */
  const void* q;
  const void* k;
  const void* v;
  const void* k2;              /* may be NULL when Sk2 == 0 */
  const void* v2;
  void* out;                   /* (B,H,Sq,D) out_dtype */
  float* lse;                  /* (B,H,Sq) fp32, may be NULL */
  xdit_strides q_stride, k_stride, v_stride, k2_stride, v2_stride, out_stride;
  int64_t lse_stride_b, lse_stride_h;   /* lse stride over Sq is 1 */
  const float* q_descale;      /* FP8 only: (B,H) fp32 each; NULL means 1.0 */
  const float* k_descale;
  const float* v_descale;
  int64_t descale_stride_b, descale_stride_h;
  void* workspace;             /* optional scratch, 16-byte aligned; may be NULL (see below) */
  int64_t workspace_bytes;
  void* stream;                /* hipStream_t; NULL = the null stream */
} xdit_attn_args;

int xdit_attn_fwd(const xdit_attn_args* args);

/*
 * Scratch bytes with which xdit_attn_fwd can balance this problem over the chip: when the number
 * of query tiles is not a multiple of what the GPU holds at once, the key/value range of the
 * tiles of the last, partly filled round is shared between workgroups, whose partial
 * (out, lse) pairs go through the workspace and are folded by the workgroups themselves at their
 * ends (tiles of up to 16 parts) or by a second small kernel.
 * Returns 0 when nothing would be gained, a negative xdit_status for invalid arguments
 * (pointers are not inspected).  Passing no or too small a workspace to xdit_attn_fwd is always
 * valid: the launch is then simply not balanced.  The workspace needs no initialisation and may
 * be used for anything else between calls (see workspace_preserved for what a caller gains by
 * leaving it alone).  No counterpart in the reference (its kernels are vendor code).
 */
int64_t xdit_attn_workspace_bytes(const xdit_attn_args* args);

/*
 * xdit_attn_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same arguments, results and kernels, but
 * the scratch of the balanced launch is a fixed array of XDIT_ATTN_NOALLOC_SCRATCH_BYTES inside
 * the library (one copy per GPU, held until the process ends) instead of a workspace of the
 * caller; args->workspace is ignored.  Nothing is allocated or freed by the call.  A problem whose
 * xdit_attn_workspace_bytes exceeds the array is rejected with XDIT_ERR_INVALID_ARG (use
 * xdit_attn_fwd with a workspace then, or set args->balance = 1: the plain launch needs no
 * scratch); Flux-1024 (B=1, H=24, S=4608, D=128) needs 28.75 MB.
 * Every call on a GPU shares that GPU's array: calls that may overlap on one GPU (two streams,
 * two threads) race on it and must be serialised by the caller; calls on one stream are ordered.
 * The array needs no clearing between calls (the kernels of a call leave its counters at zero; after
 * a call that failed a small launch clears them first).  It costs every GPU that the process uses
 * the library on its XDIT_ATTN_NOALLOC_SCRATCH_BYTES of device memory from the moment the library is
 * loaded, whether or not this entry point is ever called.  The first call on a device looks up the
 * array's device address and sets a kernel attribute: make it outside any stream capture; later
 * calls only launch kernels.  No counterpart in the reference.
 */
#define XDIT_ATTN_NOALLOC_SCRATCH_BYTES (32 * 1024 * 1024)
int xdit_attn_fwd_noalloc(const xdit_attn_args* args);

/*
 * How xdit_attn_fwd (or, with plan->ring_step set, xdit_attn_fwd_accumulate) would launch this
 * problem when given the workspace it asks for (pointers of `args` are not inspected): for tests,
 * tuning and capacity planning.  The query rows are cut
 * into `query_tiles` tiles of `rows_per_workgroup` rows, each with `kv_iterations` tiles of 64
 * keys.  `whole_tiles` of them are run by one workgroup each; with ranges > 0 the KV iterations
 * of the other tiles, laid end to end, are cut into `ranges` ranges of `range_len` iterations
 * (the last one shorter) that go to `claimers` workgroups: workgroup ids first_claimer ..
 * first_claimer + claimers - 1, of which those below whole_tiles run a whole tile first; claimer
 * c starts with range c and, with counter != 0, takes further ranges from a counter in the
 * workspace.  A query tile's partial results occupy at most `slots_per_tile` workspace slots.
 * bf16 / fp16 (head_dim up to 128; the geometry is that of head_dim 64 or 128, whichever is
 * the next one up) and fp8 (head_dim 128 or 64).  fp32 (head_dim up to 128): whole tiles only, of 128
 * rows with `kv_iterations` tiles of 32 keys, or, when those would leave more than a quarter of
 * the compute units without a workgroup, of 64 rows with tiles of 64 keys.  No counterpart in the
 * reference.
 */
typedef struct {
  uint32_t struct_size;        /* = sizeof(xdit_launch_plan), set by the caller */
  int32_t rows_per_workgroup;
  int32_t query_tiles;
  int32_t kv_iterations;
  int64_t workspace_bytes;     /* = xdit_attn_workspace_bytes(args); with ring_step: what xdit_attn_fwd_accumulate asks for */
  int32_t whole_tiles;
  int32_t ranges;
  int32_t range_len;
  int32_t slots_per_tile;
  int32_t claimers;
  int32_t first_claimer;
  int32_t counter;
  int32_t workgroups;          /* grid of the attention kernel */
  int32_t streamed;            /* != 0: streamed sharing instead of ranges: the `claimers` workgroups are dealt
                                  out over the shared tiles in contiguous groups; every member owns
                                  `range_len` KV iterations of its tile and draws the others one at a
                                  time from the tile's counter (only with streamed_sharing != 0) */
  int32_t fold_in_kernel;      /* != 0: the parts of a shared tile are folded by the workgroups of the attention
                                  kernel themselves (the ring step; tiles of at most 16 parts); 0: by a second
                                  small kernel */
  int32_t parts_first;         /* != 0: a claimer processes its range BEFORE its whole tile, and the workgroups
                                  fold the shared tiles at their ends, a slice of rows each */
  int32_t ring_step;           /* INPUT, set by the caller like struct_size: != 0 plans the launch of
                                  xdit_attn_fwd_accumulate for these arguments, 0 that of xdit_attn_fwd */
} xdit_launch_plan;

int xdit_attn_launch_plan(const xdit_attn_args* args, xdit_launch_plan* plan);

/*
 * One fold of the ring online-softmax merge, in fp32:
 *     acc_out <- acc_out - sigmoid(block_lse - acc_lse) * (acc_out - block_out)
 *     acc_lse <- acc_lse - logsigmoid(acc_lse - block_lse)
 * `first != 0` initialises instead: acc_out <- float(block_out), acc_lse <- block_lse.
 * If final_out != NULL the merged row is also written there in final_dtype (the epilogue cast
 * `out.to(q.dtype)`).  acc_out/block_out/final_out are logical (B,H,S,D); acc_lse/block_lse are
 * logical (B,H,S) with their own B/H/S strides, so the (B,S,H,1) accumulator layout of the legacy
 * ring and the (B,H,S) layout a kernel returns both map without copies.  head_dim: a multiple of
 * 8 up to 512.
 * Replaces: update_out_and_lse at ring_flash_attn.py:138, the epilogue at :145, and
 * torch _SDPAMerger._merge_one (…/_context_parallel/_attention.py:161-163, :181-182).
 */
typedef struct {
  uint32_t struct_size;        /* = sizeof(xdit_merge_args) */
  int32_t block_dtype;         /* xdit_dtype of block_out: bf16, fp16 or fp32 */
  int32_t final_dtype;         /* xdit_dtype of final_out (ignored when final_out == NULL) */
  int32_t first;               /* != 0: initialise the accumulator from the block */
  int32_t B, H, D;
  int32_t reserved0;
  int64_t S;
  float* acc_out;              /* fp32 */
  float* acc_lse;              /* fp32 */
  const void* block_out;
  const float* block_lse;      /* fp32 */
  void* final_out;             /* may be NULL */
  xdit_strides acc_out_stride, block_out_stride, final_out_stride;
  xdit_strides acc_lse_stride, block_lse_stride;
  void* stream;
} xdit_merge_args;

int xdit_lse_merge(const xdit_merge_args* args);

/*
 * One ring step in one launch: the forward of xdit_attn_fwd on this step's keys/values, folded
 * into the fp32 accumulator (acc_out, acc_lse) in the kernel's epilogue with the arithmetic of
 * xdit_lse_merge.  The block's rows are rounded to `out_dtype` before the fold, as if they had gone
 * through a block_out tensor, so the result equals xdit_attn_fwd + xdit_lse_merge bit for bit
 * (when neither launch is balanced, or both cut the KV iterations of their shared query tiles the
 * same way, which xdit_attn_launch_plan shows; to rounding of the block otherwise)
 * while the block is never written to memory and the accumulator is touched once.
 *   first != 0            initialise the accumulator from this block (acc_out is not read)
 *   args->out  (or NULL)  receives the merged rows in out_dtype: the final step's cast
 *   args->lse  (or NULL)  receives the merged log-sum-exp, (B,H,Sq) with args' lse strides
 *   discard_acc_out != 0  acc_out is read but not written back (last step: `out` and acc_lse
 *                         carry the result); needs args->out
 * acc_out is logical (B,H,Sq,D) fp32, acc_lse logical (B,H,Sq) fp32 with its own strides (the
 * (B,S,H,1) accumulator of the legacy ring maps without a copy).  bf16 / fp16 / fp32 inputs with
 * head_dim a multiple of 8 up to 128, fp8 inputs with head_dim 128 or 64; XDIT_ERR_UNSUPPORTED
 * otherwise (use the two calls).
 * args->workspace (optional, as for xdit_attn_fwd; the size this call asks for is the
 * workspace_bytes of xdit_attn_launch_plan with ring_step = 1, which can differ from
 * xdit_attn_workspace_bytes because the ring step is planned on its own; a smaller buffer is
 * valid, the launch is then not balanced) lets the launch be balanced: the parts of the shared
 * query tiles are then folded, and folded on into the accumulator, by the attention kernel's own
 * workgroups, and the result still equals a balanced xdit_attn_fwd with the same ranges +
 * xdit_lse_merge bit for bit.
 * Replaces, per ring step: the kernel call at ring_flash_attn.py:123-134, update_out_and_lse at
 * :138 and, on the last step, the cast at :145.
 */
typedef struct {
  uint32_t struct_size;        /* = sizeof(xdit_ring_acc) */
  int32_t first;
  int32_t discard_acc_out;
  int32_t reserved0;
  float* acc_out;
  float* acc_lse;
  xdit_strides acc_out_stride, acc_lse_stride;
} xdit_ring_acc;

int xdit_attn_fwd_accumulate(const xdit_attn_args* args, const xdit_ring_acc* acc);

/*
 * Abs-max fp8 quantiser, the step in front of the fp8 forward:
 *     scale = absmax(x) / 448 (1.0 if x is all zero) ;  y = fp8_e4m3fn(x / scale) ;  descale = scale
 * `per_tensor != 0`: one abs-max over the whole tensor, broadcast to every (b,h) entry of
 * `descale` — the reference's per_tensor_quant (attention_backend.py:606-615), whose descale is
 * `scale.expand(B, H)`.  `per_tensor == 0`: one abs-max per (batch, head) slice.
 * `scale_in != NULL` (device pointer to one float) supplies a static scale instead of the abs-max
 * (the `scale=` argument of per_tensor_quant).  Values whose quotient exceeds 448 saturate.
 * `x2` / `y2` (S2 > 0): a second tensor (B,H,S2,D) quantised with the scales of the first, the
 * abs-max taken over both (the joint keys, or values, that a caller would otherwise torch.cat onto
 * the first tensor before quantising: usp.py:239-241 in front of attention_backend.py:606-615).
 * `scratch`: optional device memory of at least XDIT_FP8_QUANT_SCRATCH_BYTES(B, H) bytes, private
 * to the stream until the call's kernels finish, no initialisation needed.  With it the call is
 * two launches (abs-max with one scratch slot per workgroup; cast), one with a static scale.
 * Without it `descale` (B*H contiguous fp32) doubles as the reduction buffer and the call is four
 * launches (clear, abs-max through atomics, cast, descales); results are the same.
 * `hadamard_block` (0 or 1 = off; else a power of two <= 128 that divides D) first rotates every
 * row along head_dim, block by block, by the orthonormal Sylvester-Hadamard matrix R of that size
 * with entries +-r, r = 1/sqrt(block) rounded to in_dtype, and rounds the result to in_dtype:
 * `torch.matmul(x.unflatten(-1, (D/block, block)), R).flatten(-2)` of the reference's
 * _fp8_hadamard_rotate (attention_backend.py:703-714; matrix :71-94).  Applied to both q and k
 * it leaves q.k unchanged and spreads outliers before the fp8 cast (:725-728).
 */
typedef struct {
  uint32_t struct_size;        /* = sizeof(xdit_quant_args) */
  int32_t in_dtype;            /* bf16, fp16 or fp32 */
  int32_t per_tensor;
  int32_t B, H, D;
  int64_t S;
  const void* x;               /* (B,H,S,D) in_dtype */
  void* y;                     /* (B,H,S,D) fp8 e4m3fn bytes */
  float* descale;              /* (B,H) fp32, contiguous */
  const float* scale_in;       /* optional static scale, may be NULL */
  xdit_strides x_stride, y_stride;
  void* stream;
  int32_t hadamard_block;
  int32_t reserved0;
  int64_t S2;                  /* rows of the second tensor (0 = none) */
  const void* x2;              /* (B,H,S2,D) in_dtype */
  void* y2;                    /* (B,H,S2,D) fp8 e4m3fn bytes */
  xdit_strides x2_stride, y2_stride;
  void* scratch;               /* optional, may be NULL */
  int64_t scratch_bytes;
} xdit_quant_args;

#define XDIT_FP8_QUANT_SCRATCH_BYTES(B, H) (4 * ((int64_t)(B) * (H) > 4096 ? (int64_t)(B) * (H) : 4096))

int xdit_fp8_quant(const xdit_quant_args* args);

/*
 * Pre-attention prologue of an xDiT attention processor, fused into one pass over Q (or K):
 *     y = rotary(norm(x)), written through its own strides (e.g. BSHD in, BHSD-contiguous out)
 * replacing `attn.norm_q(query)`, `apply_rotary_emb(query, image_rotary_emb)` and the later
 * `.transpose(1, 2)` + contiguous copy (transformer_flux.py:116-147,
 * transformer_hunyuan_video.py:48-83, transformer_wan.py:99-122 under
 * xfuser/model_executor/models/transformers/).  With norm and rotation off it is a strided
 * re-layout (what V needs).  x and y are logical (B,H,S,D) with element strides.
 *   norm   XDIT_NORM_NONE; XDIT_NORM_HEAD: RMSNorm over head_dim of every (b,h,s) row, `weight`
 *          has D entries; XDIT_NORM_TOKEN: over all H*D elements of a token, `weight` has H*D
 *          entries indexed h*D+d (Wan's norm over the un-split projection).  Statistics in fp32:
 *          x * rsqrt(mean(x^2) + eps), rounded to dtype, times weight (same dtype; NULL = no
 *          gain), rounded again: the roundings of diffusers' RMSNorm with a 16-bit gain.
 *   rope   XDIT_ROPE_NONE; XDIT_ROPE_INTERLEAVED: pairs (2i, 2i+1),
 *          out[j] = x[j] cos[j] + rot[j] sin[j] with rot = (-x[2i+1], x[2i]) (diffusers
 *          apply_rotary_emb, use_real_unbind_dim=-1); XDIT_ROPE_SPLIT_HALF: pairs (j, j + D/2)
 *          (use_real_unbind_dim=-2); XDIT_ROPE_WAN: out[2i] = x[2i] cos[2i] - x[2i+1] sin[2i+1],
 *          out[2i+1] = x[2i] sin[2i+1] + x[2i+1] cos[2i] (transformer_wan.py:108-120).
 *          cos / sin are fp32, `rope_stride` elements from row to row, D values per row, shared
 *          by batch and heads.  Only sequence rows [rope_row0, rope_row0 + rope_rows) are
 *          rotated, with table row s - rope_row0 (HunyuanVideo rotates the video tokens and not
 *          the text tokens behind them); products in fp32, result rounded to dtype.
 */
enum xdit_norm_mode { XDIT_NORM_NONE = 0, XDIT_NORM_HEAD = 1, XDIT_NORM_TOKEN = 2 };
enum xdit_rope_mode { XDIT_ROPE_NONE = 0, XDIT_ROPE_INTERLEAVED = 1, XDIT_ROPE_SPLIT_HALF = 2, XDIT_ROPE_WAN = 3 };

typedef struct {
  uint32_t struct_size;        /* = sizeof(xdit_prologue_args) */
  int32_t dtype;               /* bf16, fp16 or fp32: x, y and weight */
  int32_t norm;                /* xdit_norm_mode */
  int32_t rope;                /* xdit_rope_mode */
  int32_t B, H, D;
  float eps;
  int64_t S;
  const void* x;
  void* y;
  const void* weight;          /* may be NULL */
  const float* cos;            /* NULL when rope == XDIT_ROPE_NONE */
  const float* sin;
  int64_t rope_stride;
  int64_t rope_row0, rope_rows;
  xdit_strides x_stride, y_stride;
  void* stream;
} xdit_prologue_args;

int xdit_qk_prologue(const xdit_prologue_args* args);

/*
 * `count` (1..8) prologue jobs in ONE launch: the Q, K and V tensors of the text and image streams
 * of an attention block (what transformer_flux.py:116-147 handles with some ten separate torch
 * kernels).  All jobs share dtype and stream; XDIT_NORM_TOKEN jobs cannot be batched.
 */
int xdit_qk_prologue_batch(const xdit_prologue_args* jobs, int32_t count);

/* Message of the last error on the calling thread ("" if none). Never NULL. */
const char* xdit_attn_last_error(void);

/* XDIT_ATTN_ABI_VERSION the library was built with. */
int xdit_attn_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* XDIT_AMD_ATTN_H */
