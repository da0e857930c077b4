"""Switching a real xDiT install to the MI355X kernels by name.

xDiT resolves the attention function per call from `ATTENTION_FUNCTION_REGISTRY`, a dict keyed by
`AttentionBackendType` members (xfuser/core/distributed/attention_backend.py:23, :429-463; lookup in
xfuser/model_executor/layers/usp.py:205-216; the member is chosen by name in
xfuser/core/distributed/runtime_state.py:113-131 and :173-203).  A Python Enum cannot grow members
after it is created, so without editing xDiT the way in is to take over existing members:

    import xdit_amd.plugin
    xdit_amd.plugin.install()                      # AITER -> bf16/fp16 kernel, AITER_FP8 -> fp8 kernel
    # then run xDiT with --attention_backend aiter  (or aiter_fp8)

`install` returns the functions it replaced so `uninstall` can put them back.  With the two-line
patch that adds `MI355` / `MI355_FP8` members to the enum, pass `names={"MI355": ..., ...}`.
"""
from .attention_backend import _mi355_attn_call, _mi355_fp8_attn_call

DEFAULT_NAMES = {"AITER": _mi355_attn_call, "AITER_FP8": _mi355_fp8_attn_call}


def _adapt(func):
    """The registry prototype is (query, key, value, dropout_p, is_causal, attention_kwargs=None);
    xDiT's own joint decorator concatenates the joint keys/values before calling it."""
    def call(query, key, value, dropout_p, is_causal, attention_kwargs=None):
        return func(query, key, value, dropout_p, is_causal, attention_kwargs=attention_kwargs)
    call.__name__ = func.__name__
    call.__doc__ = func.__doc__
    return call


def install(backend_module=None, names=None):
    """Register the MI355X adapters in xDiT's registry under the given enum member names.
    `backend_module` is xfuser.core.distributed.attention_backend (imported when omitted)."""
    if backend_module is None:
        import importlib
        backend_module = importlib.import_module("xfuser.core.distributed.attention_backend")
    enum = backend_module.AttentionBackendType
    registry = backend_module.ATTENTION_FUNCTION_REGISTRY
    replaced = {}
    for name, func in (names or DEFAULT_NAMES).items():
        try:
            member = enum[name.upper()]
        except KeyError:
            raise ValueError(f"Value '{name}' is not a valid attention backend.") from None
        replaced[member] = registry.get(member)
        registry[member] = _adapt(func)
    return replaced


def uninstall(replaced, backend_module=None):
    """Put back what `install` replaced."""
    if backend_module is None:
        import importlib
        backend_module = importlib.import_module("xfuser.core.distributed.attention_backend")
    registry = backend_module.ATTENTION_FUNCTION_REGISTRY
    for member, func in replaced.items():
        if func is None:
            registry.pop(member, None)
        else:
            registry[member] = func
