"""Attention-backend plugin surface (registry form).

Mirrors xfuser/core/distributed/attention_backend.py: an enum of backends, a decorator registry
(:23, :456-463) and adapters with the prototype
    func(query, key, value, dropout_p, is_causal, attention_kwargs=None) -> (out, lse)
on BHSD tensors (:504-516 for the prototype, :774-823 for what HIP devices run today).
The two adapters here call the gfx950 kernels through the C ABI.  Unlike the reference's AITER
adapter (:780-782) nothing is permuted or made contiguous: the kernels take BHSD strides.
"""
from enum import Enum

import torch

from . import custom_ops  # noqa: F401  (registers torch.ops.xdit_amd.*)
from . import ops

ATTENTION_FUNCTION_REGISTRY = {}


class AttentionBackendType(Enum):
    MI355 = "MI355X HIP"
    MI355_FP8 = "MI355X HIP FP8"


def register_attention_function(backend_type):
    """Decorator to register attention functions with their corresponding backend type."""
    def decorator(func):
        ATTENTION_FUNCTION_REGISTRY[backend_type] = func
        return func
    return decorator


# attention_kwargs keys the reference's other backends consume and this one does not implement
_UNSUPPORTED_KWARGS = (
    "attn_mask", "indices_k", "cu_seqlens_k", "max_seqlen_k",  # key-padding / varlen (:465-489)
    "tile_size", "thw", "block_mask",                           # block-sparse backends
)


def _check_call(dropout_p, is_causal, attention_kwargs):
    if dropout_p not in (0, 0.0, None):
        raise ValueError(f"dropout_p={dropout_p} is not supported (inference path: dropout_p must be 0.0)")
    if is_causal:
        raise NotImplementedError("is_causal=True is not implemented: DiT attention is non-causal")
    if attention_kwargs:
        for key in _UNSUPPORTED_KWARGS:
            if attention_kwargs.get(key) is not None:
                raise NotImplementedError(f"attention_kwargs['{key}'] is not supported by the MI355X backend")


def _split_joint(key, value, joint_kv):
    """joint_kv = (joint_key, joint_value, strategy): order the two KV segments the way the
    reference's torch.cat does (usp.py:179-189): "rear" -> [kv, joint], "front" -> [joint, kv]."""
    if joint_kv is None:
        return key, value, None, None
    joint_key, joint_value, strategy = joint_kv
    if strategy == "rear":
        return key, value, joint_key, joint_value
    if strategy == "front":
        return joint_key, joint_value, key, value
    raise ValueError(f"Invalid joint_strategy: {strategy}")


@register_attention_function(AttentionBackendType.MI355)
def _mi355_attn_call(query, key, value, dropout_p, is_causal, attention_kwargs=None, joint_kv=None):
    """bf16 / fp16 / fp32 attention; softmax scale is D**-0.5 as on the reference's AITER path
    (attention_backend.py:790).  Returns (out BHSD in query's dtype, lse (B,H,S) fp32)."""
    _check_call(dropout_p, is_causal, attention_kwargs)
    k1, v1, k2, v2 = _split_joint(key, value, joint_kv)
    scale = query.shape[-1] ** -0.5
    if torch.compiler.is_compiling():
        # under torch.compile the call goes through the registered custom ops (fake
        # implementations describe the outputs, so tracing does not break the graph)
        if k2 is None:
            return torch.ops.xdit_amd.attn_fwd(query, k1, v1, scale)
        return torch.ops.xdit_amd.attn_fwd_joint(query, k1, v1, k2, v2, scale)
    return ops.attn_fwd(query, k1, v1, softmax_scale=scale, k2=k2, v2=v2)


def get_dtype_max(dtype):
    try:
        return torch.finfo(dtype).max
    except TypeError:
        return torch.iinfo(dtype).max


# Block size of the Hadamard rotation the fp8 adapter applies to q and k before quantising, as the
# reference's AITER fp8 adapter does with a 128x128 matrix (attention_backend.py:374, :725-728).
# 0 switches it off (the reference's FLASH_3_FP8 adapter, :617-642, does not rotate).
FP8_HADAMARD_BLOCK = 128


def per_tensor_quant(x, scale=None, scale_dtype=torch.float32, quant_dtype=torch.float8_e4m3fn, dtypeMax=None,
                     hadamard_block=0):
    """Same contract as the reference's per_tensor_quant (attention_backend.py:606-615):
    one abs-max scale over the whole tensor, y = fp8(x / scale), descale expanded to x.shape[:2].
    With `scale=None` the abs-max reduction and the cast run in the HIP quantiser.
    `hadamard_block` fuses _fp8_hadamard_rotate (:703-714) in front: x is rotated along head_dim
    in blocks of that size before the abs-max and the cast."""
    if quant_dtype != torch.float8_e4m3fn:
        raise NotImplementedError("only float8_e4m3fn (the fp8 format of gfx950) is supported")
    if scale is None and dtypeMax in (None, get_dtype_max(quant_dtype)):
        if torch.compiler.is_compiling():
            y, descale = torch.ops.xdit_amd.fp8_quant(x, True, hadamard_block)
        else:
            y, descale = ops.fp8_quant(x, per_tensor=True, hadamard_block=hadamard_block)
        return y, descale.to(scale_dtype)
    if scale is None:
        if hadamard_block > 1:
            raise NotImplementedError("a non-default dtypeMax together with the fused rotation is not implemented")
        scale = torch.abs(x.to(torch.float32)).max() / dtypeMax
    scale = torch.as_tensor(scale, dtype=torch.float32, device=x.device)
    y, descale = ops.fp8_quant(x, per_tensor=True, scale=scale, hadamard_block=hadamard_block)
    return y, descale.to(scale_dtype)


@register_attention_function(AttentionBackendType.MI355_FP8)
def _mi355_fp8_attn_call(query, key, value, dropout_p, is_causal, attention_kwargs=None, joint_kv=None):
    """fp8 attention: quantise q, k, v per tensor (as _flash_attn_3_fp8_call :617-642 and
    _aiter_fp8_attn_call :717-772 do), run the fp8 kernel with (B,H) descales, return a bf16/fp16
    output in the query's dtype AND the lse (the reference's AITER fp8 path returns no lse, :732).
    q and k are Hadamard-rotated along head_dim inside the quantiser (block FP8_HADAMARD_BLOCK, or
    attention_kwargs["hadamard_block"]; 0 = off), as the AITER fp8 adapter does (:725-728).
    Inputs that are already float8_e4m3fn take their descales from attention_kwargs
    ("q_descale", "k_descale", "v_descale")."""
    _check_call(dropout_p, is_causal, attention_kwargs)
    if joint_kv is not None:
        key = torch.cat([key, joint_kv[0]] if joint_kv[2] == "rear" else [joint_kv[0], key], dim=2)
        value = torch.cat([value, joint_kv[1]] if joint_kv[2] == "rear" else [joint_kv[1], value], dim=2)
    scale = query.shape[-1] ** -0.5
    if query.dtype == torch.float8_e4m3fn:
        kw = attention_kwargs or {}
        return ops.attn_fwd(query, key, value, softmax_scale=scale, q_descale=kw.get("q_descale"),
                            k_descale=kw.get("k_descale"), v_descale=kw.get("v_descale"),
                            out_dtype=kw.get("out_dtype", torch.bfloat16))
    out_dtype = query.dtype if query.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    had = (attention_kwargs or {}).get("hadamard_block", FP8_HADAMARD_BLOCK)
    if had > 1 and query.shape[-1] % had != 0:
        had = 0
    # rotating q and k alike leaves q.k unchanged and spreads outliers before the fp8 cast
    q8, qd = per_tensor_quant(query, hadamard_block=had)
    k8, kd = per_tensor_quant(key, hadamard_block=had)
    v8, vd = per_tensor_quant(value)
    if torch.compiler.is_compiling():
        return torch.ops.xdit_amd.attn_fwd_fp8(q8, k8, v8, qd, kd, vd, scale, out_dtype == torch.float16)
    return ops.attn_fwd(q8, k8, v8, softmax_scale=scale, q_descale=qd, k_descale=kd, v_descale=vd, out_dtype=out_dtype)
