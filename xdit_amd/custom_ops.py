"""`torch.library` custom ops over the HIP entry points, so `torch.compile` can trace through them.

The reference wraps a vendor kernel the same way (xfuser/core/distributed/attention_backend.py:383-399:
`@custom_op("xfuser::flydsl_attn_kernel", mutates_args=())` plus a `register_fake` that returns
`torch.empty_like(query)`).  Here every op has a device implementation that calls the C ABI
(`xdit_amd.ops`) and a fake implementation that only describes the outputs:

    xdit_amd::attn_fwd        (q, k, v, softmax_scale)                      -> (out, lse)
    xdit_amd::attn_fwd_joint  (q, k, v, k2, v2, softmax_scale)              -> (out, lse)
    xdit_amd::attn_fwd_fp8    (q, k, v, q_descale, k_descale, v_descale,
                               softmax_scale, out_fp16)                     -> (out, lse)
    xdit_amd::lse_merge       (acc_out, acc_lse, block_out, block_lse, first)   in place
    xdit_amd::lse_merge_final (acc_out, acc_lse, block_out, block_lse, final_out)  in place
    xdit_amd::attn_fwd_fp8_joint (q, k, v, k2, v2, q_descale, k_descale, v_descale,
                               softmax_scale, out_fp16)                     -> (out, lse)
    xdit_amd::attn_fwd_accumulate (q, k, v, k2?, v2?, acc_out, acc_lse, final_out?, first,
                               discard_acc_out, softmax_scale)              in place (one ring step)
    xdit_amd::fp8_quant       (x, per_tensor, hadamard_block)               -> (y, descale)
    xdit_amd::fp8_quant_ex    (x, x2?, scale?, per_tensor, hadamard_block)  -> (y, y2, descale)
    xdit_amd::norm_rope       (x, weight, cos, sin, eps, norm, rope,
                               rope_row0, rope_rows)                        -> y (BHSD-contiguous)

All tensors are logical BHSD (any B/H/S strides); outputs are BHSD-contiguous, lse is (B,H,Sq)
fp32.  The ops are registered for GPU tensors only: there is no CPU implementation.
"""
from typing import Optional, Tuple

import torch
from torch.library import custom_op, register_fake

from . import ops

Tensor = torch.Tensor


def _fake_out_lse(query: Tensor, out_dtype) -> Tuple[Tensor, Tensor]:
    B, H, Sq, D = query.shape
    return (query.new_empty((B, H, Sq, D), dtype=out_dtype),
            query.new_empty((B, H, Sq), dtype=torch.float32))


@custom_op("xdit_amd::attn_fwd", mutates_args=(), device_types="cuda")
def attn_fwd(query: Tensor, key: Tensor, value: Tensor, softmax_scale: float) -> Tuple[Tensor, Tensor]:
    return ops.attn_fwd(query, key, value, softmax_scale=softmax_scale)


@register_fake("xdit_amd::attn_fwd")
def _attn_fwd_fake(query, key, value, softmax_scale):
    return _fake_out_lse(query, query.dtype)


@custom_op("xdit_amd::attn_fwd_joint", mutates_args=(), device_types="cuda")
def attn_fwd_joint(query: Tensor, key: Tensor, value: Tensor, key2: Tensor, value2: Tensor,
                   softmax_scale: float) -> Tuple[Tensor, Tensor]:
    return ops.attn_fwd(query, key, value, softmax_scale=softmax_scale, k2=key2, v2=value2)


@register_fake("xdit_amd::attn_fwd_joint")
def _attn_fwd_joint_fake(query, key, value, key2, value2, softmax_scale):
    return _fake_out_lse(query, query.dtype)


@custom_op("xdit_amd::attn_fwd_fp8", mutates_args=(), device_types="cuda")
def attn_fwd_fp8(query: Tensor, key: Tensor, value: Tensor, q_descale: Tensor, k_descale: Tensor,
                 v_descale: Tensor, softmax_scale: float, out_fp16: bool) -> Tuple[Tensor, Tensor]:
    return ops.attn_fwd(query, key, value, softmax_scale=softmax_scale, q_descale=q_descale,
                        k_descale=k_descale, v_descale=v_descale,
                        out_dtype=torch.float16 if out_fp16 else torch.bfloat16)


@register_fake("xdit_amd::attn_fwd_fp8")
def _attn_fwd_fp8_fake(query, key, value, q_descale, k_descale, v_descale, softmax_scale, out_fp16):
    return _fake_out_lse(query, torch.float16 if out_fp16 else torch.bfloat16)


@custom_op("xdit_amd::attn_fwd_fp8_joint", mutates_args=(), device_types="cuda")
def attn_fwd_fp8_joint(query: Tensor, key: Tensor, value: Tensor, key2: Tensor, value2: Tensor, q_descale: Tensor,
                       k_descale: Tensor, v_descale: Tensor, softmax_scale: float, out_fp16: bool) -> Tuple[Tensor, Tensor]:
    return ops.attn_fwd(query, key, value, softmax_scale=softmax_scale, k2=key2, v2=value2, q_descale=q_descale,
                        k_descale=k_descale, v_descale=v_descale,
                        out_dtype=torch.float16 if out_fp16 else torch.bfloat16)


@register_fake("xdit_amd::attn_fwd_fp8_joint")
def _attn_fwd_fp8_joint_fake(query, key, value, key2, value2, q_descale, k_descale, v_descale, softmax_scale, out_fp16):
    return _fake_out_lse(query, torch.float16 if out_fp16 else torch.bfloat16)


@custom_op("xdit_amd::attn_fwd_accumulate", mutates_args=("acc_out", "acc_lse", "final_out"), device_types="cuda")
def attn_fwd_accumulate(query: Tensor, key: Tensor, value: Tensor, key2: Optional[Tensor], value2: Optional[Tensor],
                        acc_out: Tensor, acc_lse: Tensor, final_out: Optional[Tensor], first: bool,
                        discard_acc_out: bool, softmax_scale: float) -> None:
    """One ring step (`ops.attn_fwd_accumulate`): the block of (key, value) [+ (key2, value2)] folded
    into the fp32 accumulator in the attention kernel's epilogue; `final_out` also receives the
    merged rows in the query's dtype."""
    ops.attn_fwd_accumulate(query, key, value, acc_out, acc_lse, first=first, final_out=final_out,
                            discard_acc_out=discard_acc_out, softmax_scale=softmax_scale, k2=key2, v2=value2)


@register_fake("xdit_amd::attn_fwd_accumulate")
def _attn_fwd_accumulate_fake(query, key, value, key2, value2, acc_out, acc_lse, final_out, first, discard_acc_out, softmax_scale):
    return None


@custom_op("xdit_amd::lse_merge", mutates_args=("acc_out", "acc_lse"), device_types="cuda")
def lse_merge(acc_out: Tensor, acc_lse: Tensor, block_out: Tensor, block_lse: Tensor, first: bool) -> None:
    ops.lse_merge(acc_out, acc_lse, block_out, block_lse, first=first)


@register_fake("xdit_amd::lse_merge")
def _lse_merge_fake(acc_out, acc_lse, block_out, block_lse, first):
    return None


@custom_op("xdit_amd::lse_merge_final", mutates_args=("acc_out", "acc_lse", "final_out"), device_types="cuda")
def lse_merge_final(acc_out: Tensor, acc_lse: Tensor, block_out: Tensor, block_lse: Tensor, final_out: Tensor) -> None:
    ops.lse_merge(acc_out, acc_lse, block_out, block_lse, first=False, final_out=final_out)


@register_fake("xdit_amd::lse_merge_final")
def _lse_merge_final_fake(acc_out, acc_lse, block_out, block_lse, final_out):
    return None


@custom_op("xdit_amd::fp8_quant", mutates_args=(), device_types="cuda")
def fp8_quant(x: Tensor, per_tensor: bool, hadamard_block: int) -> Tuple[Tensor, Tensor]:
    return ops.fp8_quant(x, per_tensor=per_tensor, hadamard_block=hadamard_block)


@register_fake("xdit_amd::fp8_quant")
def _fp8_quant_fake(x, per_tensor, hadamard_block):
    B, H, S, D = x.shape
    return (x.new_empty((B, H, S, D), dtype=torch.float8_e4m3fn),
            x.new_empty((B, H), dtype=torch.float32))


@custom_op("xdit_amd::fp8_quant_ex", mutates_args=(), device_types="cuda")
def fp8_quant_ex(x: Tensor, x2: Optional[Tensor], scale: Optional[Tensor], per_tensor: bool,
                 hadamard_block: int) -> Tuple[Tensor, Tensor, Tensor]:
    """`ops.fp8_quant` with its optional second tensor (quantised with the scales of the first) and
    its optional static scale (a one-element fp32 tensor).  Without `x2` the second result has no rows."""
    out = ops.fp8_quant(x, per_tensor=per_tensor, scale=scale, hadamard_block=hadamard_block, x2=x2)
    if x2 is None:
        B, H, _, D = x.shape
        return out[0], x.new_empty((B, H, 0, D), dtype=torch.float8_e4m3fn), out[1]
    return out


@register_fake("xdit_amd::fp8_quant_ex")
def _fp8_quant_ex_fake(x, x2, scale, per_tensor, hadamard_block):
    B, H, S, D = x.shape
    S2 = 0 if x2 is None else x2.shape[2]
    return (x.new_empty((B, H, S, D), dtype=torch.float8_e4m3fn),
            x.new_empty((B, H, S2, D), dtype=torch.float8_e4m3fn),
            x.new_empty((B, H), dtype=torch.float32))


@custom_op("xdit_amd::norm_rope", mutates_args=(), device_types="cuda")
def norm_rope(x: Tensor, weight: Tensor, cos: Tensor, sin: Tensor, eps: float, norm: str, rope: str,
              rope_row0: int, rope_rows: int) -> Tensor:
    """Fused RMSNorm + rotary embedding + re-layout of a logical BHSD tensor (`ops.qk_prologue`).
    `norm` is "none", "head" or "token" (`weight` is ignored for "none": pass any tensor);
    `rope` is "none", "interleaved", "split_half" or "wan" (`cos`/`sin` ignored for "none")."""
    return ops.qk_prologue(x, weight=None if norm == "none" else weight, eps=eps, norm=None if norm == "none" else norm,
                           rotary_emb=None if rope == "none" else (cos, sin), rope="interleaved" if rope == "none" else rope,
                           rope_row0=rope_row0, rope_rows=rope_rows if rope != "none" else None)


@register_fake("xdit_amd::norm_rope")
def _norm_rope_fake(x, weight, cos, sin, eps, norm, rope, rope_row0, rope_rows):
    return x.new_empty(tuple(x.shape))
