"""CPU oracle for the attention hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU in float64 (or float32 where noted), the arithmetic of the
reference's single-device attention path.  Only `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py` may import it; the product (`xdit_amd/`) never does.

What each function follows (paths relative to the xDiT source tree unless prefixed `torch:`,
which is the PyTorch wheel the reference depends on):

* `attn_fwd_ref`         softmax(Q K^T * scale) V and logsumexp, the contract of the registry
                         adapters xfuser/core/distributed/attention_backend.py:504-516 (out, lse),
                         :518-532 (math path, out only), :774-823 (AITER: scale = D**-0.5).
* `merge_ref`            torch:distributed/tensor/experimental/_context_parallel/_attention.py:181-182
                         (the sigmoid / logsigmoid form; yunchang's update_out_and_lse, reached at
                         xfuser/core/long_ctx_attention/ring/ring_flash_attn.py:138, is the same).
* `update_out_and_lse_ref`  first-call and layout semantics visible at ring_flash_attn.py:68-69,
                         :138, :145-148 (BSHD accumulator, lse kept as (B,S,H,1)).
* `ring_forward_ref`     the loop of ring_flash_attn.py:83-148 on one device (KV chunks visited
                         in the order a rank would receive them), joint K/V on the first ("front")
                         or last ("rear") step, :89-100.
* `per_tensor_quant_ref` attention_backend.py:606-615.
* `hadamard_matrix`, `hadamard_rotate_ref`  attention_backend.py:71-94 (Sylvester construction,
                         1/sqrt(n) normalisation) and :703-714 (block-wise rotation of head_dim).
* `rms_norm_ref`, `apply_rotary_emb_ref`, `apply_rotary_emb_wan_ref`  the steps of the attention
                         processors in front of the attention call: transformer_flux.py:116-147,
                         transformer_hunyuan_video.py:48-83, transformer_wan.py:99-122.  The first two
                         restate diffusers (>=0.33.0, absent here) from its published source.
* `sdpa_cpu`             the body of `_sdpa_attn_call`, attention_backend.py:499-501 (used as the
                         timed CPU baseline).

Pinning (tests/test_oracle.py): brute force with math.fsum on tiny inputs; torch's own CPU
ops `aten._scaled_dot_product_attention_math` and `aten._scaled_dot_product_flash_attention_for_cpu`;
closed forms and invariants of the merge (log-add-exp identity, fold of any KV partition equals the
single pass, -inf block is the identity, equal lse gives the mean); the C twin in attn_ref.c;
for the Hadamard rotation the sign rule (-1)^popcount(i&j), orthonormality, an independent fast
Walsh-Hadamard transform, and invariance of q.k under a common rotation; for the prologue
torch's own `F.rms_norm` in float64, complex multiplication as the independent form of the
rotation, pair-norm preservation, identity at angle 0, and agreement of the three rotation
conventions on tables where they must agree.
The reference holds no golden vectors for this path, so values are pinned by those checks, and
the tolerances (not values) come from the reference's tests.
"""
import math

import numpy as np
import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------------------------
# attention forward
# ----------------------------------------------------------------------------------------------
def attn_fwd_ref(q, k, v, softmax_scale=None, dtype=torch.float64, q_chunk=1024):
    """(out, lse) for logical BHSD tensors, evaluated in `dtype` on the CPU.

    out_i = sum_j softmax_j(scale * q_i.k_j) v_j ; lse_i = log sum_j exp(scale * q_i.k_j)
    (natural log, scale included).  Query rows are processed in chunks to bound memory.
    """
    q = q.detach().to("cpu").to(dtype)
    k = k.detach().to("cpu").to(dtype)
    v = v.detach().to("cpu").to(dtype)
    B, H, Sq, D = q.shape
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    out = torch.empty((B, H, Sq, v.shape[-1]), dtype=dtype)
    lse = torch.empty((B, H, Sq), dtype=dtype)
    kt = k.transpose(-1, -2)
    for s0 in range(0, Sq, q_chunk):
        s = torch.matmul(q[:, :, s0:s0 + q_chunk], kt) * softmax_scale
        m = s.max(dim=-1, keepdim=True).values
        p = torch.exp(s - m)
        l = p.sum(dim=-1, keepdim=True)
        out[:, :, s0:s0 + q_chunk] = torch.matmul(p, v) / l
        lse[:, :, s0:s0 + q_chunk] = (m + torch.log(l)).squeeze(-1)
    return out, lse


def attn_rows_ref(q, k, v, rows, softmax_scale=None, dtype=torch.float64):
    """(out, lse) for the given query rows only (all batches and heads, full K/V).
    Used to probe long sequences where the full reference is too expensive."""
    idx = torch.as_tensor(rows, dtype=torch.long)
    return attn_fwd_ref(q.detach().to("cpu")[:, :, idx], k, v, softmax_scale, dtype)


def attn_bruteforce(q, k, v, softmax_scale):
    """Pure-Python restatement with exactly rounded sums (math.fsum) for tiny inputs.
    q: [Sq][D], k: [Sk][D], v: [Sk][Dv] nested lists of floats -> (out [Sq][Dv], lse [Sq])."""
    out, lse = [], []
    for qi in q:
        s = [softmax_scale * math.fsum(a * b for a, b in zip(qi, kj)) for kj in k]
        m = max(s)
        e = [math.exp(x - m) for x in s]
        l = math.fsum(e)
        lse.append(m + math.log(l))
        out.append([math.fsum(e[j] * v[j][d] for j in range(len(k))) / l for d in range(len(v[0]))])
    return out, lse


def sdpa_cpu(q, k, v):
    """What the reference's default SDPA adapter runs (attention_backend.py:499-501), on CPU."""
    return F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False)


# ----------------------------------------------------------------------------------------------
# ring merge
# ----------------------------------------------------------------------------------------------
def merge_ref(out, lse, block_out, block_lse, dtype=torch.float64):
    """One fold.  out/block_out: (..., D); lse/block_lse: (...) (no trailing 1).
    out' = out - sigmoid(block_lse - lse) * (out - block_out)
    lse' = lse - logsigmoid(lse - block_lse)"""
    out = out.to(dtype)
    block_out = block_out.to(dtype)
    lse = lse.to(dtype).unsqueeze(-1)
    block_lse = block_lse.to(dtype).unsqueeze(-1)
    new_out = out - torch.sigmoid(block_lse - lse) * (out - block_out)
    new_lse = lse - F.logsigmoid(lse - block_lse)
    return new_out, new_lse.squeeze(-1)


def merge_closed_form(out, lse, block_out, block_lse):
    """The same fold written as the log-add-exp identity (float64):
    L = log(e^l1 + e^l2), o = (e^l1 o1 + e^l2 o2) / e^L."""
    l1 = lse.double().unsqueeze(-1)
    l2 = block_lse.double().unsqueeze(-1)
    L = torch.logaddexp(l1, l2)
    o = torch.exp(l1 - L) * out.double() + torch.exp(l2 - L) * block_out.double()
    return o, L.squeeze(-1)


def update_out_and_lse_ref(out, lse, block_out, block_lse, dtype=torch.float32):
    """The legacy ring's accumulator update in its own layout: block_out (B,S,H,D),
    block_lse (B,H,S); accumulator out fp32 (B,S,H,D), lse fp32 (B,S,H,1).
    First call (out is None) initialises from the block."""
    if out is None:
        return block_out.to(dtype), block_lse.to(dtype).transpose(-2, -1).unsqueeze(-1)
    bl = block_lse.to(dtype).transpose(-2, -1).unsqueeze(-1)
    bo = block_out.to(dtype)
    new_out = out - torch.sigmoid(bl - lse) * (out - bo)
    new_lse = lse - F.logsigmoid(lse - bl)
    return new_out, new_lse


def ring_forward_ref(q, k, v, n_chunks, order=None, softmax_scale=None, joint_k=None, joint_v=None,
                     joint_strategy="none", chunk_dtype=None, dtype=torch.float64):
    """Single-device restatement of the ring loop on BHSD tensors: K/V are split into `n_chunks`
    contiguous chunks visited in `order` (default: the order rank 0 sees, [0, P-1, ..., 1]); each
    step's (out_i, lse_i) is folded with `merge_ref`.  `chunk_dtype` optionally rounds each
    per-chunk output (as a bf16 kernel would) before the fold."""
    P = n_chunks
    if order is None:
        order = [0] + list(range(P - 1, 0, -1))
    ks = k.chunk(P, dim=2)
    vs = v.chunk(P, dim=2)
    out = lse = None
    for step, c in enumerate(order):
        kk, vv = ks[c], vs[c]
        if joint_strategy == "front" and step == 0:
            kk, vv = torch.cat([joint_k, kk], 2), torch.cat([joint_v, vv], 2)
        elif joint_strategy == "rear" and step == P - 1:
            kk, vv = torch.cat([kk, joint_k], 2), torch.cat([vv, joint_v], 2)
        bo, bl = attn_fwd_ref(q, kk, vv, softmax_scale, dtype)
        if chunk_dtype is not None:
            bo = bo.to(chunk_dtype).to(dtype)
            bl = bl.float().to(dtype)
        if out is None:
            out, lse = bo, bl
        else:
            out, lse = merge_ref(out, lse, bo, bl, dtype)
    return out, lse


# ----------------------------------------------------------------------------------------------
# fp8
# ----------------------------------------------------------------------------------------------
FP8_MAX = 448.0  # torch.finfo(torch.float8_e4m3fn).max


def per_tensor_quant_ref(x, scale=None):
    """attention_backend.py:606-615: scale = absmax(x)/448 over the WHOLE tensor, y = fp8(x/scale),
    descale broadcast to x.shape[:2]."""
    x = x.to(torch.float32)
    if scale is None:
        scale = torch.abs(x).max() / FP8_MAX
    y = x / scale
    return y.to(torch.float8_e4m3fn), scale.expand(*x.shape[:2]).to(torch.float32)


def per_head_quant_ref(x):
    """Per-(batch, head) abs-max quantiser for a BHSD tensor: scale[b,h] = absmax(x[b,h])/448
    (1.0 for an all-zero slice)."""
    x = x.to(torch.float32)
    amax = x.abs().amax(dim=(2, 3))
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    y = (x / scale[:, :, None, None]).to(torch.float8_e4m3fn)
    return y, scale


def hadamard_matrix(block_r, dtype=torch.float64):
    """Orthonormal Sylvester-Hadamard matrix: H1=[[1]], H2n=[[Hn,Hn],[Hn,-Hn]], divided by
    sqrt(block_r) in float32 and then cast to `dtype` (attention_backend.py:86-94, the construction
    the reference falls back to and the normalisation it applies at :85)."""
    assert block_r > 0 and (block_r & (block_r - 1)) == 0
    H = torch.ones((1, 1), dtype=torch.float32)
    while H.shape[0] < block_r:
        H = torch.cat([torch.cat([H, H], dim=1), torch.cat([H, -H], dim=1)], dim=0)
    return (H / (block_r ** 0.5)).to(dtype)


def hadamard_rotate_ref(x, block_r):
    """_fp8_hadamard_rotate (attention_backend.py:703-714): x @ R along head_dim in blocks of
    block_r, R held in x's dtype, result in x's dtype.  The products are summed in float64 here
    (a matmul sums them in fp32 in an unspecified order), then rounded once to x's dtype."""
    d = x.shape[-1]
    R = hadamard_matrix(block_r, x.dtype).to(torch.float64)
    xb = x.to(torch.float64).unflatten(-1, (d // block_r, block_r))
    return torch.matmul(xb, R).flatten(-2).to(x.dtype)


def dequant(y, scale):
    """fp8 bytes + (B,H) scales -> float32 BHSD."""
    return y.to(torch.float32) * scale[:, :, None, None].to(torch.float32)


# ----------------------------------------------------------------------------------------------
# pre-attention prologue (RMSNorm of Q/K, rotary embedding)
# ----------------------------------------------------------------------------------------------
def rms_norm_ref(x, weight=None, eps=1e-6):
    """RMSNorm over the last dimension with the rounding points of the modules behind
    `attn.norm_q` / `attn.norm_k` (transformer_flux.py:120-121): diffusers' RMSNorm.forward
    (diffusers>=0.33.0, models/normalization.py — a dependency that is not in the reference tree;
    restated from its published source) and, with the same roundings, the in-tree
    xfuser/model_executor/models/customized/step_video_t2v/normalization.py:34-60:
        variance = x.float().pow(2).mean(-1) ; h = x * rsqrt(variance + eps)      (fp32)
        16-bit weight: h = h.to(weight.dtype) * weight ; no weight: h.to(x.dtype)."""
    input_dtype = x.dtype
    variance = x.to(torch.float32).pow(2).mean(-1, keepdim=True)
    h = x * torch.rsqrt(variance + eps)
    if weight is not None:
        if weight.dtype in (torch.float16, torch.bfloat16):
            h = h.to(weight.dtype)
        h = h * weight
    else:
        h = h.to(input_dtype)
    return h


def apply_rotary_emb_ref(x, freqs_cis, use_real_unbind_dim=-1, sequence_dim=2):
    """diffusers' apply_rotary_emb with use_real=True (models/embeddings.py of diffusers>=0.33.0,
    restated; called at transformer_flux.py:146-147 with sequence_dim=1 and at
    transformer_hunyuan_video.py:60-83 with the default 2).  x [B,H,S,D] or [B,S,H,D];
    freqs_cis = (cos, sin), each [S,D]."""
    cos, sin = freqs_cis
    if sequence_dim == 2:
        cos, sin = cos[None, None, :, :], sin[None, None, :, :]
    elif sequence_dim == 1:
        cos, sin = cos[None, :, None, :], sin[None, :, None, :]
    else:
        raise ValueError(sequence_dim)
    if use_real_unbind_dim == -1:
        x_real, x_imag = x.reshape(*x.shape[:-1], -1, 2).unbind(-1)
        x_rotated = torch.stack([-x_imag, x_real], dim=-1).flatten(3)
    elif use_real_unbind_dim == -2:
        x_real, x_imag = x.reshape(*x.shape[:-1], 2, -1).unbind(-2)
        x_rotated = torch.cat([-x_imag, x_real], dim=-1)
    else:
        raise ValueError(use_real_unbind_dim)
    return (x.float() * cos + x_rotated.float() * sin).to(x.dtype)


def apply_rotary_emb_wan_ref(hidden_states, freqs_cos, freqs_sin):
    """The local function of transformer_wan.py:108-120 ([B,S,H,D] input, [1,S,1,D] tables)."""
    x1, x2 = hidden_states.unflatten(-1, (-1, 2)).unbind(-1)
    cos = freqs_cos[..., 0::2]
    sin = freqs_sin[..., 1::2]
    out = torch.empty_like(hidden_states)
    out[..., 0::2] = x1 * cos - x2 * sin
    out[..., 1::2] = x1 * sin + x2 * cos
    return out.type_as(hidden_states)


def rope_tables(S, D, seed=0, axes=(16, 56, 56), theta=10000.0, interleave=True):
    """Synthetic (cos, sin) tables [S, D] fp32 of the shape the DiT position embedders produce:
    per axis a of width d_a, angle = pos_a * theta^(-2i/d_a); each angle repeated for the two
    elements of its pair (`interleave`, the use_real_unbind_dim=-1 convention) or the table
    repeated for the two halves (-2).  Positions are random integers per token and axis."""
    g = torch.Generator().manual_seed(seed)
    assert sum(axes) == D or axes == ()
    if not axes:
        axes = (D,)
    cols = []
    for d_a in axes:
        pos = torch.randint(0, 64, (S,), generator=g).to(torch.float64)
        freqs = 1.0 / (theta ** (torch.arange(0, d_a, 2, dtype=torch.float64) / d_a))
        cols.append(torch.outer(pos, freqs))
    ang = torch.cat(cols, dim=1)  # [S, D/2]
    if interleave:
        ang = ang.repeat_interleave(2, dim=1)
    else:
        ang = torch.cat([ang, ang], dim=1)
    return ang.cos().float(), ang.sin().float()


# ----------------------------------------------------------------------------------------------
# seeded inputs of the benchmark configurations (generated on the CPU in fp32)
# ----------------------------------------------------------------------------------------------
def _randn(shape, gen):
    return torch.randn(shape, generator=gen, dtype=torch.float32)


def _rmsnorm_heads(x, gain, eps=1e-6):
    """Per-head RMSNorm over head_dim with one gain vector of size head_dim
    (the shape of attn.norm_q / norm_k, transformer_flux.py:120-121)."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain


def make_qkv(B, H, S, D, seed, rmsnorm=False, dtype=torch.float32):
    """q, k, v ~ N(0,1) in BHSD from `seed`; with `rmsnorm`, q and k get a per-head RMSNorm with
    gains ~ U(0.8, 1.2)."""
    g = torch.Generator().manual_seed(seed)
    q = _randn((B, H, S, D), g)
    k = _randn((B, H, S, D), g)
    v = _randn((B, H, S, D), g)
    if rmsnorm:
        gq = 0.8 + 0.4 * torch.rand(D, generator=g)
        gk = 0.8 + 0.4 * torch.rand(D, generator=g)
        q = _rmsnorm_heads(q, gq)
        k = _rmsnorm_heads(k, gk)
    return q.to(dtype), k.to(dtype), v.to(dtype)


CONFIGS = {
    # name: (B, H, S, D, seed, rmsnorm, dtype)
    "c1_pixart512": (1, 16, 1024, 72, 1001, False, torch.float32),
    "c2_flux1024": (1, 24, 4608, 128, 1002, True, torch.bfloat16),
    "c4_hunyuan720p_shard": (1, 3, 118800 + 256, 128, 1004, True, torch.bfloat16),
    "c5_wan720p_shard_fp8": (1, 5, 75600, 128, 1005, False, torch.float8_e4m3fn),
}


def make_config(name, S=None):
    """Inputs of a named configuration (optionally with a shorter sequence for CPU-sized tests).
    Returns a dict with q, k, v (and q_descale, k_descale, v_descale for fp8)."""
    B, H, S0, D, seed, rms, dtype = CONFIGS[name]
    S = S0 if S is None else S
    if dtype == torch.float8_e4m3fn:
        q, k, v = make_qkv(B, H, S, D, seed, rms, torch.float32)
        out = {}
        for n, t in (("q", q), ("k", k), ("v", v)):
            y, s = per_head_quant_ref(t)
            out[n] = y
            out[n + "_descale"] = s
        return out
    q, k, v = make_qkv(B, H, S, D, seed, rms, dtype)
    return {"q": q, "k": k, "v": v}
