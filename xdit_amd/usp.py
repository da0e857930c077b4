"""Single-device form of xDiT's USP attention entry (xfuser/model_executor/layers/usp.py).

`USP` and `attention` keep the reference's signatures (usp.py:247-262, :364-373).  On one device
the sequence-parallel world size is 1, so USP is the branch at usp.py:316-323: one backend call.
`ring_chunks > 1` additionally runs the ring schedule of usp.py:46-74 on one device: K/V are
split into chunks that are visited in the order rank 0 of a ring would receive them, and the
per-chunk (out, lse) partials are folded by `SDPAMerger` (torch's _SDPAMerger,
torch/distributed/tensor/experimental/_context_parallel/_attention.py:138-223).
"""
import functools

import torch

from . import ops
from . import attention_backend as AB
from .attention_backend import ATTENTION_FUNCTION_REGISTRY, AttentionBackendType

_DEFAULT_BACKEND = AttentionBackendType.MI355
_DECORATED = {}   # backend -> (registered function, its joint-decorated wrapper)


def set_default_backend(backend):
    """Counterpart of RuntimeState.set_attention_backend (runtime_state.py:113-131)."""
    global _DEFAULT_BACKEND
    if isinstance(backend, str):
        try:
            backend = AttentionBackendType[backend.upper()]
        except KeyError:
            raise ValueError(f"Value '{backend}' is not a valid attention backend.") from None
    if backend not in ATTENTION_FUNCTION_REGISTRY:
        raise NotImplementedError(f"Attention backend {backend} not registered.")
    _DEFAULT_BACKEND = backend


def _concat_joint_tensor(tensor, joint_tensor, joint_strategy, dim):
    """Concatenate the joint tensor to the main tensor based on the joint strategy (usp.py:179-189)."""
    if joint_strategy == "rear":
        tensor = torch.cat([tensor, joint_tensor], dim=dim)
    elif joint_strategy == "front":
        tensor = torch.cat([joint_tensor, tensor], dim=dim)
    else:
        raise ValueError(f"Invalid joint_strategy: {joint_strategy}")
    return tensor


def _get_attention_function(backend=None):
    """Registry lookup wrapped by the joint decorator (usp.py:205-216)."""
    attention_backend = backend if backend is not None else _DEFAULT_BACKEND
    func = ATTENTION_FUNCTION_REGISTRY.get(attention_backend, None)
    if func is None:
        raise NotImplementedError(f"Attention backend {attention_backend} not registered.")
    cached = _DECORATED.get(attention_backend)
    if cached is None or cached[0] is not func:   # one wrapper per registered function: ring_attn recognises it by identity
        cached = (func, concat_joint_tensors_decorator(func))
        _DECORATED[attention_backend] = cached
    return cached[1]


def concat_joint_tensors_decorator(func):
    """Same rule as usp.py:218-245: the joint (text) keys/values take part on ring step 0 for
    "front" and on the last step for "rear", and `step` is incremented in place.  Instead of
    torch.cat-ing them onto K and V (a copy of the whole K and V), they are handed to the kernel
    as a second KV segment."""
    @functools.wraps(func)
    def wrapper(*args, **kwargs):
        query, key, value = args[0:3]
        is_causal = kwargs.get("is_causal")
        dropout_p = kwargs.get("dropout_p")
        joint_attn_kwargs = kwargs.get("joint_attn_kwargs", None)
        attention_kwargs = kwargs.get("attention_kwargs", None)
        joint_kv = None
        if joint_attn_kwargs is not None:
            joint_strategy = joint_attn_kwargs.get("joint_strategy", None)
            joint_key = joint_attn_kwargs.get("joint_key", None)
            joint_value = joint_attn_kwargs.get("joint_value", None)
            step = joint_attn_kwargs.get("step", 0)
            total_steps = joint_attn_kwargs.get("total_steps", 1)
            if (joint_strategy == "front" and step == 0) or (joint_strategy == "rear" and step == total_steps - 1):
                joint_kv = (joint_key, joint_value, joint_strategy)
            joint_attn_kwargs["step"] = step + 1  # in place increment step
        return func(query, key, value, dropout_p=dropout_p, is_causal=is_causal,
                    attention_kwargs=attention_kwargs, joint_kv=joint_kv)
    return wrapper


class SDPAMerger:
    """Fold of per-chunk (out, lse) partials in BHSD, fp32 accumulators (torch _SDPAMerger:
    first block stored :161-163, later blocks merged :181-182, results cast back :215-223).
    Each step is one fused HIP pass; `results()` of the last step's cast is fused into that pass
    when `final_step=True` is given to `step`."""

    def __init__(self):
        self._out = None
        self._lse = None
        self._final = None
        self._out_dtype = torch.float32

    def step(self, out, lse, final_step=False):
        self._out_dtype = out.dtype
        first = self._out is None
        if first:
            self._out = torch.empty(out.shape, dtype=torch.float32, device=out.device)
            self._lse = torch.empty(lse.shape, dtype=torch.float32, device=out.device)
        final = None
        if final_step and out.dtype != torch.float32:
            final = torch.empty(out.shape, dtype=out.dtype, device=out.device)
        if torch.compiler.is_compiling():   # the registered custom ops (traceable)
            if final is None:
                torch.ops.xdit_amd.lse_merge(self._out, self._lse, out, lse, first)
            else:
                torch.ops.xdit_amd.lse_merge_final(self._out, self._lse, out, lse, final)
        else:
            ops.lse_merge(self._out, self._lse, out, lse, first=first, final_out=final)
        self._final = final

    def results(self):
        assert self._out is not None and self._lse is not None
        out = self._final if self._final is not None else self._out.to(self._out_dtype)
        return out, self._lse


def ring_attn(attention_function, query, key, value, dropout_p=0.0, is_causal=False,
              joint_attn_kwargs=None, attention_kwargs=None, ring_chunks=1, order=None):
    """The ring schedule of usp.py:46-74 on one device.  K/V are split into `ring_chunks`
    contiguous chunks; `order` defaults to what rank 0 sees: [0, P-1, P-2, ..., 1]."""
    P = ring_chunks
    if key.shape[2] % P != 0:
        raise ValueError(f"key length {key.shape[2]} is not divisible by ring_chunks={P}")
    if order is None:
        order = [0] + list(range(P - 1, 0, -1))
    k_chunks = key.chunk(P, dim=2)
    v_chunks = value.chunk(P, dim=2)
    mi355 = ATTENTION_FUNCTION_REGISTRY.get(AttentionBackendType.MI355)
    decorated = _DECORATED.get(AttentionBackendType.MI355)
    ours = attention_function is mi355 or (decorated is not None and decorated[0] is mi355 and attention_function is decorated[1])
    if P > 1 and ops.fused_ring_step_supported(query) and ours:
        # every step is one launch: the kernel folds its block into the accumulator itself (same
        # bits as the call + merge below); the joint keys/values join on the step the decorator
        # would pick
        AB._check_call(dropout_p, is_causal, attention_kwargs)
        acc_out = torch.empty(query.shape, dtype=torch.float32, device=query.device)
        acc_lse = torch.empty(query.shape[:3], dtype=torch.float32, device=query.device)
        final = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        for i, c in enumerate(order):
            joint_kv = None
            if joint_attn_kwargs is not None:
                strategy = joint_attn_kwargs.get("joint_strategy", None)
                step = joint_attn_kwargs.get("step", 0)
                if (strategy == "front" and step == 0) or (strategy == "rear" and step == joint_attn_kwargs.get("total_steps", 1) - 1):
                    joint_kv = (joint_attn_kwargs.get("joint_key", None), joint_attn_kwargs.get("joint_value", None), strategy)
                joint_attn_kwargs["step"] = step + 1
            k1, v1, k2, v2 = AB._split_joint(k_chunks[c], v_chunks[c], joint_kv)
            last = i == P - 1
            if torch.compiler.is_compiling():   # the same call as a registered custom op (traceable)
                torch.ops.xdit_amd.attn_fwd_accumulate(query, k1, v1, k2, v2, acc_out, acc_lse, final if last else None,
                                                       i == 0, last, query.shape[-1] ** -0.5)
            else:
                ops.attn_fwd_accumulate(query, k1, v1, acc_out, acc_lse, first=i == 0,
                                        final_out=final if last else None, discard_acc_out=last,
                                        softmax_scale=query.shape[-1] ** -0.5, k2=k2, v2=v2)
        return final
    merger = SDPAMerger()
    for i, c in enumerate(order):
        out, lse = attention_function(query, k_chunks[c], v_chunks[c], dropout_p=dropout_p, is_causal=is_causal,
                                      joint_attn_kwargs=joint_attn_kwargs, attention_kwargs=attention_kwargs)
        merger.step(out, lse, final_step=(i == P - 1))
    return merger.results()[0]


def USP(query, key, value, dropout_p=0.0, is_causal=False, joint_query=None, joint_key=None,
        joint_value=None, joint_strategy=None, attn_layer=None, combine_qkv_a2a=None, backend=None,
        attention_kwargs=None, head_balance_layer=None, ring_chunks=1):
    """USP attention call on one device; BHSD in, BHSD out (usp.py:247-361).

    `attn_layer` (PipeFusion KV cache), `combine_qkv_a2a` and `head_balance_layer` belong to the
    multi-GPU / sparse paths: a KV-cache layer is rejected, the other two are no-ops here exactly
    as they are in the reference when the Ulysses world size is 1."""
    if attn_layer is not None:
        raise NotImplementedError("attn_layer (PipeFusion KV cache) is not supported on the single-device path")
    attention_function = _get_attention_function(backend=backend)
    joint_attn_kwargs = None
    if joint_strategy:
        query = _concat_joint_tensor(query, joint_query, joint_strategy, dim=2)
        joint_attn_kwargs = {
            "joint_value": joint_value,
            "joint_key": joint_key,
            "joint_strategy": joint_strategy,
            "step": 0,
            "total_steps": ring_chunks,
        }
    if ring_chunks == 1:
        out, _ = attention_function(query, key, value, dropout_p=dropout_p, is_causal=is_causal,
                                    joint_attn_kwargs=joint_attn_kwargs, attention_kwargs=attention_kwargs)
    else:
        out = ring_attn(attention_function, query, key, value, dropout_p=dropout_p, is_causal=is_causal,
                        joint_attn_kwargs=joint_attn_kwargs, attention_kwargs=attention_kwargs,
                        ring_chunks=ring_chunks)
    return out


def attention(query, key, value, dropout_p=0.0, is_causal=False, backend=None, attention_kwargs=None,
              head_balance_layer=None):
    """Runs the attention call without any parallelism (usp.py:364-392)."""
    attention_function = _get_attention_function(backend=backend)
    out, _ = attention_function(query, key, value, dropout_p=dropout_p, is_causal=is_causal,
                                attention_kwargs=attention_kwargs)
    return out
