"""Pre-attention steps of xDiT's attention processors, on the fused HIP prologue.

The processors in xfuser/model_executor/models/transformers/ run, between the QKV projections and
the attention call, a per-head RMSNorm of Q and K, a rotary embedding and a transpose to BHSD as
separate torch kernels (transformer_flux.py:116-147, 170-172; transformer_hunyuan_video.py:48-83;
transformer_wan.py:99-122).  The functions here keep the call surfaces of the pieces they replace
(diffusers' `apply_rotary_emb`, an RMSNorm module's forward) and add fused forms that do all of
it in one pass and write straight into the BHSD tensor the attention kernel reads, text and image
streams side by side (no torch.cat).
"""
import threading

import torch

from . import ops


def _as_bhsd(x, sequence_dim):
    if x.ndim != 4:
        raise ValueError("expected a 4-D tensor")
    if sequence_dim == 2:
        return x
    if sequence_dim == 1:
        return x.transpose(1, 2)
    raise ValueError(f"`sequence_dim={sequence_dim}` but should be 1 or 2.")


def apply_rotary_emb(x, freqs_cis, use_real=True, use_real_unbind_dim=-1, sequence_dim=2):
    """diffusers' apply_rotary_emb (models/embeddings.py) as the processors call it
    (transformer_flux.py:146-147 with sequence_dim=1, transformer_hunyuan_video.py:60-83 with the
    default 2): x is [B,H,S,D] (sequence_dim=2) or [B,S,H,D] (1), freqs_cis = (cos, sin) of [S,D]
    fp32.  Returns a new contiguous tensor of x's shape and dtype."""
    if not use_real:
        raise NotImplementedError("complex freqs_cis (use_real=False) is not implemented")
    if use_real_unbind_dim == -1:
        rope = "interleaved"
    elif use_real_unbind_dim == -2:
        rope = "split_half"
    else:
        raise ValueError(f"`use_real_unbind_dim={use_real_unbind_dim}` but should be -1 or -2.")
    xb = _as_bhsd(x, sequence_dim)
    out = torch.empty_like(x, memory_format=torch.contiguous_format)
    ops.qk_prologue(xb, rotary_emb=freqs_cis, rope=rope, out=_as_bhsd(out, sequence_dim))
    return out


def apply_rotary_emb_wan(hidden_states, freqs_cos, freqs_sin):
    """The local function of transformer_wan.py:108-120: hidden_states [B,S,H,D], freqs [1,S,1,D]."""
    out = torch.empty_like(hidden_states, memory_format=torch.contiguous_format)
    ops.qk_prologue(hidden_states.transpose(1, 2), rotary_emb=(freqs_cos, freqs_sin), rope="wan", out=out.transpose(1, 2))
    return out


class RMSNorm(torch.nn.Module):
    """RMSNorm over the last dimension with the forward of the modules behind `attn.norm_q` /
    `attn.norm_k` (diffusers' RMSNorm; same roundings as the in-tree
    xfuser/model_executor/models/customized/step_video_t2v/normalization.py:34-60):
    x * rsqrt(mean(x^2) + eps) in fp32, rounded to the dtype, times the gain."""

    def __init__(self, dim, eps=1e-6, elementwise_affine=True, device=None, dtype=None):
        super().__init__()
        self.dim, self.eps = dim, eps
        self.weight = torch.nn.Parameter(torch.ones(dim, device=device, dtype=dtype)) if elementwise_affine else None

    def forward(self, hidden_states):
        x = hidden_states
        if x.shape[-1] != self.dim:
            raise ValueError("last dimension %d != %d" % (x.shape[-1], self.dim))
        if self.dim > 512:
            # a norm over the un-split projection (all heads of a token): rows of H*D elements
            raise NotImplementedError("use norm_rope(..., norm='token') for a norm across heads")
        rows = x.reshape(1, 1, -1, self.dim)
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        w = None if self.weight is None else self.weight.detach()
        ops.qk_prologue(rows, weight=w, eps=self.eps, norm="head", out=out.view(1, 1, -1, self.dim))
        return out


def norm_rope(x, weight=None, eps=1e-6, freqs_cis=None, sequence_dim=1, norm="head", rope="interleaved",
              rope_row0=0, rope_rows=None, out=None, out_row0=0):
    """norm -> rotary embedding -> BHSD in ONE pass.  x is the head-split projection output
    [B,S,H,D] (sequence_dim=1) or [B,H,S,D] (2).  Writes rows [out_row0, out_row0 + S) of `out`
    ([B,H,S_total,D]; a new BHSD-contiguous tensor of S rows when omitted) and returns `out`."""
    xb = _as_bhsd(x, sequence_dim)
    B, H, S, D = xb.shape
    if out is None:
        out = torch.empty((B, H, S, D), dtype=x.dtype, device=x.device)
        out_row0 = 0
    dst = out[:, :, out_row0:out_row0 + S]
    ops.qk_prologue(xb, weight=weight, eps=eps, norm=norm, rotary_emb=freqs_cis, rope=rope,
                    rope_row0=rope_row0, rope_rows=rope_rows, out=dst)
    return out


_TLS = threading.local()   # cached argument structs are patched in place: one set per thread


def flux_joint_qkv(query, key, value, encoder_query, encoder_key, encoder_value, heads,
                   norm_q, norm_k, norm_added_q, norm_added_k, image_rotary_emb, eps=1e-6):
    """Lines 116-147 and 170-172 of xFuserFluxAttnProcessor.__call__ (transformer_flux.py): head
    split, per-head RMSNorm of the image and text Q/K with their own gains, [text; image]
    concatenation along the sequence, rotary embedding over the joint sequence, transpose to
    BHSD.  Inputs are the projection outputs [B,S_img,H*D] and [B,S_txt,H*D]; norm_* are the gain
    vectors (D entries, the tensors' dtype); image_rotary_emb = (cos, sin) of [S_txt+S_img, D].
    Returns q, k, v as BHSD-contiguous [B,H,S_txt+S_img,D]: ONE launch of six jobs, no intermediate tensor."""
    srcs = (encoder_query, query, encoder_key, key, encoder_value, value)
    gains = (norm_added_q, norm_q, norm_added_k, norm_k)
    cos, sin = image_rotary_emb
    # The six argument structs are filled once per call signature (shapes, strides, dtype, device)
    # and kept; a later call only allocates the outputs and patches pointers and the stream.
    sig = (heads, float(eps), query.dtype, query.device, cos.dtype, cos.shape, cos.stride(), sin.shape, sin.stride(),
           tuple((t.shape, t.stride()) for t in srcs), tuple(None if g is None else (g.shape, g.stride(), g.dtype) for g in gains))
    plans = _TLS.__dict__.setdefault("flux_plans", {})
    plan = plans.get(sig)
    B, S_img, HD = query.shape
    S_txt = encoder_query.shape[1]
    D = HD // heads
    outs = tuple(torch.empty((B, heads, S_txt + S_img, D), dtype=query.dtype, device=query.device) for _ in range(3))
    if plan is None:
        jobs = []
        for t, (txt, img) in enumerate(((encoder_query, query), (encoder_key, key), (encoder_value, value))):
            for src, w, row0 in ((txt, gains[2 * t] if t < 2 else None, 0), (img, gains[2 * t + 1] if t < 2 else None, S_txt)):
                xb = src.unflatten(-1, (heads, D)).transpose(1, 2)
                n = xb.shape[2]
                job = dict(x=xb, out=outs[t][:, :, row0:row0 + n])
                if t < 2:
                    job.update(weight=w, eps=eps, norm="head", rotary_emb=(cos[row0:row0 + n], sin[row0:row0 + n]),
                               rope="interleaved")
                jobs.append(job)
        arr = ops.prologue_batch_args(jobs)
        # where each pointer of each job lies relative to the tensor it comes from
        plan = (arr, [(arr[i].y - outs[i // 2].data_ptr(),
                       arr[i].cos - cos.data_ptr() if arr[i].cos else None,
                       arr[i].sin - sin.data_ptr() if arr[i].sin else None,
                       gains[i] is not None and arr[i].weight == gains[i].data_ptr() if i < 4 else False) for i in range(6)])
        if len(plans) >= 64:
            plans.clear()
        # a gain or table that had to be copied (not contiguous) cannot be patched by pointer: no plan then
        if (cos.is_contiguous() and sin.is_contiguous()
                and all(rec[3] or (i >= 4 or gains[i] is None) for i, rec in enumerate(plan[1]))):
            plans[sig] = plan
    else:
        arr, recs = plan
        cp, sp = cos.data_ptr(), sin.data_ptr()
        for i in range(6):
            a = arr[i]
            y_off, c_off, s_off, has_w = recs[i]
            a.x = srcs[i].data_ptr()
            a.y = outs[i // 2].data_ptr() + y_off
            if c_off is not None:
                a.cos, a.sin = cp + c_off, sp + s_off
            if has_w:
                a.weight = gains[i].data_ptr()
    ops.launch_prologue_batch(arr, 6, query.device)
    return outs
