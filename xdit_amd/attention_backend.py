"""Attention-backend plugin surface (registry form).

Mirrors xfuser/core/distributed/attention_backend.py: an enum of backends, a decorator registry
(:23, :456-463) and adapters with the prototype
    func(query, key, value, dropout_p, is_causal, attention_kwargs=None) -> (out, lse)
on BHSD tensors (:504-516 for the prototype, :774-823 for what HIP devices run today).
The two adapters here call the gfx950 kernels through the C ABI.  Unlike the reference's AITER
adapter (:780-782) nothing is permuted or made contiguous: the kernels take BHSD strides.
"""
import os
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


# Static scale of the fp8 adapter for q, k and v alike, as the reference's AITER fp8 adapter takes
# one from XFUSER_AITER_FP8_STATIC_SCALE_WITH_DESCALE (attention_backend.py:735-745); None = dynamic
# (abs-max) scaling.  attention_kwargs["fp8_static_scale"] overrides it per call.
_env_scale = os.environ.get("XFUSER_AITER_FP8_STATIC_SCALE_WITH_DESCALE")
FP8_STATIC_SCALE = float(_env_scale) if _env_scale not in (None, "") else None


def per_tensor_quant(x, scale=None, scale_dtype=torch.float32, quant_dtype=torch.float8_e4m3fn, dtypeMax=None,
                     hadamard_block=0, x2=None):
    """Same contract as the reference's per_tensor_quant (attention_backend.py:606-615):
    one abs-max scale over the whole tensor, y = fp8(x / scale), descale expanded to x.shape[:2].
    With `scale=None` the abs-max reduction and the cast run in the HIP quantiser.
    `hadamard_block` fuses _fp8_hadamard_rotate (:703-714) in front: x is rotated along head_dim
    in blocks of that size before the abs-max and the cast.  `x2` (the joint keys or values) is
    quantised with the same scale, the abs-max taken over both tensors as if they had been
    concatenated first; the result is then (y, y2, descale)."""
    if quant_dtype != torch.float8_e4m3fn:
        raise NotImplementedError("only float8_e4m3fn (the fp8 format of gfx950) is supported")
    compiling = torch.compiler.is_compiling()   # then through the registered custom ops (fake implementations describe the outputs)

    def quant(scale_tensor):
        if compiling:
            y, y2, descale = torch.ops.xdit_amd.fp8_quant_ex(x, x2, scale_tensor, True, hadamard_block)
            out = (y, descale) if x2 is None else (y, y2, descale)
        else:
            out = ops.fp8_quant(x, per_tensor=True, scale=scale_tensor, hadamard_block=hadamard_block, x2=x2)
        return (*out[:-1], out[-1].to(scale_dtype))

    if scale is None and dtypeMax in (None, get_dtype_max(quant_dtype)):
        return quant(None)
    if scale is None:
        if hadamard_block > 1 or x2 is not None:
            raise NotImplementedError("a non-default dtypeMax together with the fused rotation or a second tensor is not implemented")
        scale = torch.abs(x.to(torch.float32)).max() / dtypeMax
    scale = torch.as_tensor(scale, dtype=torch.float32, device=x.device).reshape(1)
    return quant(scale)


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
    kw = attention_kwargs or {}
    scale = query.shape[-1] ** -0.5
    jk = jv = strategy = None
    if joint_kv is not None:
        jk, jv, strategy = joint_kv
        if strategy not in ("front", "rear"):
            raise ValueError(f"Invalid joint_strategy: {strategy}")
    if query.dtype == torch.float8_e4m3fn:
        k1, v1, k2, v2 = _split_joint(key, value, joint_kv)
        return ops.attn_fwd(query, k1, v1, softmax_scale=scale, k2=k2, v2=v2, q_descale=kw.get("q_descale"),
                            k_descale=kw.get("k_descale"), v_descale=kw.get("v_descale"),
                            out_dtype=kw.get("out_dtype", torch.bfloat16))
    out_dtype = query.dtype if query.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    had = kw.get("hadamard_block", FP8_HADAMARD_BLOCK)
    if had > 1 and query.shape[-1] % had != 0:
        had = 0
    static = kw.get("fp8_static_scale", FP8_STATIC_SCALE)
    # rotating q and k alike leaves q.k unchanged and spreads outliers before the fp8 cast
    q8, qd = per_tensor_quant(query, scale=static, hadamard_block=had)
    if jk is None:
        k8, kd = per_tensor_quant(key, scale=static, hadamard_block=had)
        v8, vd = per_tensor_quant(value, scale=static)
        k2 = v2 = None
    else:
        # the joint keys / values share the scale of the keys / values they are attended with (one
        # abs-max over both, as quantising their concatenation would give) and go to the kernel as
        # its second KV segment: no concatenated copy of K and V is made
        k8, k2, kd = per_tensor_quant(key, scale=static, hadamard_block=had, x2=jk)
        v8, v2, vd = per_tensor_quant(value, scale=static, x2=jv)
        if strategy == "front":
            k8, v8, k2, v2 = k2, v2, k8, v8
    if torch.compiler.is_compiling():
        if k2 is None:
            return torch.ops.xdit_amd.attn_fwd_fp8(q8, k8, v8, qd, kd, vd, scale, out_dtype == torch.float16)
        return torch.ops.xdit_amd.attn_fwd_fp8_joint(q8, k8, v8, k2, v2, qd, kd, vd, scale, out_dtype == torch.float16)
    return ops.attn_fwd(q8, k8, v8, softmax_scale=scale, k2=k2, v2=v2, q_descale=qd, k_descale=kd, v_descale=vd,
                        out_dtype=out_dtype)
