"""Host-side logic of the reference-shaped call surfaces, checked on the CPU (no kernels run):
argument domains, the joint-tensor step rule, ring ordering, registry behaviour, and that
nothing falls back to a CPU implementation."""
import pytest
import torch

from xdit_amd import attention_backend as AB
from xdit_amd import ops, ring, usp


def test_registry_and_lookup():
    assert AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355] is AB._mi355_attn_call
    assert AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355_FP8] is AB._mi355_fp8_attn_call
    with pytest.raises(NotImplementedError):
        usp._get_attention_function(backend="nope")

    @AB.register_attention_function("custom")
    def f(q, k, v, dropout_p, is_causal, attention_kwargs=None, joint_kv=None):
        return q, None
    try:
        assert AB.ATTENTION_FUNCTION_REGISTRY["custom"] is f
        assert usp.attention(torch.ones(1), None, None, backend="custom") is not None
    finally:
        del AB.ATTENTION_FUNCTION_REGISTRY["custom"]


def test_argument_domain_matches_reference_call_sites():
    q = torch.zeros(1, 2, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        AB._mi355_attn_call(q, q, q, 0.1, False)
    with pytest.raises(NotImplementedError):
        AB._mi355_attn_call(q, q, q, 0.0, True)
    with pytest.raises(NotImplementedError):
        AB._mi355_attn_call(q, q, q, 0.0, False, attention_kwargs={"attn_mask": torch.ones(1)})
    with pytest.raises(NotImplementedError):
        AB._mi355_attn_call(q, q, q, 0.0, False, attention_kwargs={"indices_k": torch.ones(1)})
    qb = q.transpose(1, 2)
    for kw in (dict(causal=True), dict(window_size=(3, 3)), dict(softcap=1.0), dict(alibi_slopes=torch.ones(2))):
        with pytest.raises(NotImplementedError):
            ring.flash_attn_forward(qb, qb, qb, **kw)
    with pytest.raises(ValueError):
        ring.flash_attn_forward(qb, qb, qb, dropout_p=0.5)


def test_no_cpu_fallback():
    """CPU tensors must fail loudly: the product has no path other than the HIP library."""
    q = torch.zeros(1, 2, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.attn_fwd(q, q, q)
    with pytest.raises(RuntimeError, match="no CPU path"):
        usp.USP(q, q, q)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.lse_merge(torch.zeros(1, 2, 4, 128), torch.zeros(1, 2, 4), q, torch.zeros(1, 2, 4))


def test_shape_and_dtype_validation():
    q = torch.zeros(1, 2, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.attn_fwd(q[0], q, q)
    with pytest.raises(ValueError):
        ops.attn_fwd(q, q, q, k2=q)  # k2 without v2


def test_joint_decorator_step_rule():
    """front -> joint K/V on step 0 only; rear -> on the last step only; step incremented in place
    (the rule of usp.py:218-245)."""
    calls = []

    def fake(q, k, v, dropout_p, is_causal, attention_kwargs=None, joint_kv=None):
        calls.append(joint_kv)
        return q, None
    f = usp.concat_joint_tensors_decorator(fake)
    for strategy, expect in (("front", [True, False, False]), ("rear", [False, False, True])):
        calls.clear()
        kw = {"joint_key": "jk", "joint_value": "jv", "joint_strategy": strategy, "step": 0, "total_steps": 3}
        for _ in range(3):
            f("q", "k", "v", dropout_p=0.0, is_causal=False, joint_attn_kwargs=kw)
        assert [c is not None for c in calls] == expect
        assert kw["step"] == 3
        assert [c for c in calls if c is not None][0] == ("jk", "jv", strategy)
    calls.clear()
    f("q", "k", "v", dropout_p=0.0, is_causal=False)
    assert calls == [None]


def test_joint_segment_order_matches_cat_order():
    assert AB._split_joint("k", "v", ("jk", "jv", "rear")) == ("k", "v", "jk", "jv")
    assert AB._split_joint("k", "v", ("jk", "jv", "front")) == ("jk", "jv", "k", "v")
    with pytest.raises(ValueError):
        AB._split_joint("k", "v", ("jk", "jv", "middle"))
    with pytest.raises(ValueError):
        usp._concat_joint_tensor(torch.ones(1), torch.ones(1), "middle", 0)
    a, b = torch.zeros(1, 1, 2, 1), torch.ones(1, 1, 1, 1)
    assert usp._concat_joint_tensor(a, b, "rear", 2).flatten().tolist() == [0, 0, 1]
    assert usp._concat_joint_tensor(a, b, "front", 2).flatten().tolist() == [1, 0, 0]


def test_local_ring_order():
    assert ring.LocalRing(4).order() == [0, 3, 2, 1]      # what rank 0 of a 4-ring receives
    assert ring.LocalRing(4, rank=2).order() == [2, 1, 0, 3]
    assert ring.LocalRing(1).order() == [0]
    with pytest.raises(ValueError):
        ring.LocalRing(0)


def test_legacy_ring_argument_errors():
    q = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="simultaneously"):
        ring.xdit_ring_flash_attn_forward(None, q, q, q, 0.1, causal=False, joint_tensor_key=q)
    with pytest.raises(ValueError, match="not supprted"):
        ring.xdit_ring_flash_attn_forward(None, q, q, q, 0.1, causal=False, joint_tensor_key=q,
                                          joint_tensor_value=q, joint_strategy="none")
    with pytest.raises(ValueError, match="divisible"):
        ring.xdit_ring_flash_attn_forward(ring.LocalRing(3), q, q, q, 0.1, causal=False)
    layer = ring.xFuserLongContextAttention()
    with pytest.raises(ValueError, match="simultaneously"):
        layer(None, q, q, q, joint_tensor_query=q)
    with pytest.raises(NotImplementedError):
        ring.update_out_and_lse(None, None, q, torch.zeros(1, 2, 8), slice_=(slice(0, 1),))


def test_custom_ops_fake_implementations_describe_the_outputs():
    """The `torch.library` ops (pattern of attention_backend.py:383-399 in the reference) must
    trace on meta tensors: shapes, dtypes and contiguity of what the kernels return."""
    from xdit_amd import custom_ops  # noqa: F401
    B, H, Sq, Sk, D = 2, 3, 40, 70, 128
    # BSHD memory viewed as BHSD, as a Flux block hands it over
    q = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="meta").transpose(1, 2)
    k = torch.empty(B, Sk, H, D, dtype=torch.bfloat16, device="meta").transpose(1, 2)
    out, lse = torch.ops.xdit_amd.attn_fwd(q, k, k, 0.1)
    assert out.shape == (B, H, Sq, D) and out.dtype == torch.bfloat16 and out.is_contiguous()
    assert lse.shape == (B, H, Sq) and lse.dtype == torch.float32
    k2 = torch.empty(B, H, 9, D, dtype=torch.bfloat16, device="meta")
    out, lse = torch.ops.xdit_amd.attn_fwd_joint(q, k, k, k2, k2, 0.1)
    assert out.shape == (B, H, Sq, D) and lse.shape == (B, H, Sq)
    q8 = torch.empty(B, H, Sq, D, dtype=torch.float8_e4m3fn, device="meta")
    k8 = torch.empty(B, H, Sk, D, dtype=torch.float8_e4m3fn, device="meta")
    d = torch.empty(B, H, device="meta")
    out, lse = torch.ops.xdit_amd.attn_fwd_fp8(q8, k8, k8, d, d, d, 0.1, True)
    assert out.dtype == torch.float16 and out.shape == (B, H, Sq, D) and lse.dtype == torch.float32
    out, _ = torch.ops.xdit_amd.attn_fwd_fp8(q8, k8, k8, d, d, d, 0.1, False)
    assert out.dtype == torch.bfloat16
    y, ds = torch.ops.xdit_amd.fp8_quant(q, False, 128)
    assert y.dtype == torch.float8_e4m3fn and y.shape == q.shape and y.is_contiguous() and ds.shape == (B, H)
    y, y2, ds = torch.ops.xdit_amd.fp8_quant_ex(k, k2, None, True, 0)
    assert y.shape == k.shape and y2.shape == k2.shape and y2.dtype == torch.float8_e4m3fn and ds.shape == (B, H)
    y, y2, ds = torch.ops.xdit_amd.fp8_quant_ex(k, None, torch.empty(1, device="meta"), True, 128)
    assert y.shape == k.shape and y2.shape == (B, H, 0, D)
    k28 = torch.empty(B, H, 9, D, dtype=torch.float8_e4m3fn, device="meta")
    out, lse = torch.ops.xdit_amd.attn_fwd_fp8_joint(q8, k8, k8, k28, k28, d, d, d, 0.1, False)
    assert out.dtype == torch.bfloat16 and out.shape == (B, H, Sq, D) and lse.shape == (B, H, Sq)
    acc = torch.empty(B, H, Sq, D, device="meta")
    assert torch.ops.xdit_amd.attn_fwd_accumulate(q, k, k, k2, k2, acc, torch.empty(B, H, Sq, device="meta"), None, True, False, 0.1) is None
    w = torch.empty(D, dtype=torch.bfloat16, device="meta")
    cs = torch.empty(Sq, D, device="meta")
    y = torch.ops.xdit_amd.norm_rope(q, w, cs, cs, 1e-6, "head", "interleaved", 0, Sq)
    assert y.shape == q.shape and y.dtype == q.dtype and y.is_contiguous()
    # there is no CPU implementation behind the ops either
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.xdit_amd.attn_fwd(torch.zeros(1, 1, 4, 128), torch.zeros(1, 1, 4, 128), torch.zeros(1, 1, 4, 128), 0.1)


def test_plugin_install_takes_over_registry_members_by_name():
    """`plugin.install` against a stand-in for xfuser.core.distributed.attention_backend (an enum
    plus a dict registry, attention_backend.py:23, :429-463)."""
    import types
    from enum import Enum
    from xdit_amd import plugin

    class AttentionBackendType(Enum):
        SDPA = "SDPA"
        AITER = "AITER"
        AITER_FP8 = "AITER FP8"

    old = lambda *a, **k: "old"
    mod = types.SimpleNamespace(AttentionBackendType=AttentionBackendType,
                                ATTENTION_FUNCTION_REGISTRY={AttentionBackendType.AITER: old})
    replaced = plugin.install(mod)
    reg = mod.ATTENTION_FUNCTION_REGISTRY
    assert reg[AttentionBackendType.AITER].__name__ == "_mi355_attn_call"
    assert reg[AttentionBackendType.AITER_FP8].__name__ == "_mi355_fp8_attn_call"
    # the installed functions have the registry prototype and the same argument domain
    q = torch.zeros(1, 2, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        reg[AttentionBackendType.AITER](q, q, q, 0.0, True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        reg[AttentionBackendType.AITER](q, q, q, 0.0, False)
    plugin.uninstall(replaced, mod)
    assert reg[AttentionBackendType.AITER] is old and AttentionBackendType.AITER_FP8 not in reg
    with pytest.raises(ValueError):
        plugin.install(mod, names={"nope": old})


def test_default_backend_by_name():
    usp.set_default_backend("mi355_fp8")
    try:
        assert usp._DEFAULT_BACKEND is AB.AttentionBackendType.MI355_FP8
        with pytest.raises(ValueError):
            usp.set_default_backend("flash_9")
    finally:
        usp.set_default_backend(AB.AttentionBackendType.MI355)


def test_bench_refuses_more_than_one_gpu_and_lists_the_model_shapes():
    """bench.py runs on one GPU only: --gpus above 1 exits with a message before touching a device;
    the table of model shapes names shapes the kernels accept (head_dim a multiple of 8 up to 128)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""
    sys.path.insert(0, root)
    import bench
    assert len(bench.MODEL_SHAPES) >= 10
    for name, B, H, Sq, Sk, D in bench.MODEL_SHAPES:
        assert D % 8 == 0 and 0 < D <= 128 and min(B, H, Sq, Sk) > 0, name
        assert ops.fused_ring_step_supported(torch.empty(1, 1, 1, D, dtype=torch.bfloat16))


