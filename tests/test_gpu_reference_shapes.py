"""The reference's own tests for this path, restated for one device.

xDiT's tests compare live GPU backends with each other and store no expected values, so what
carries over is their shapes, their structure and their tolerances:
  * tests/core/test_ring_flash_attn.py:34-165  fp16 (1, 128, 4, 32) BSHD, ring of 2 ranks against
    one-shot attention, rtol = atol = 1e-3; causal, joint "rear", joint "front".  One device plays
    every rank in turn (LocalRing(2, rank) visits the KV chunks in the order that rank would).
  * tests/layers/usp_test.py:29-190            bf16 (1, 24, 14867, 128): USP and ring_attn per
    backend against the default backend, abs difference below 0.05 (`places=1`).  The comparison
    here is the CPU oracle on probe rows plus torch's own attention on the GPU where it runs.
  * tests/layers/usp_test.py:193-265           USP against the layer form, plain and with 64 joint
    "rear" tokens, abs difference below 5e-4 (`places=3`).
"""
import pytest
import torch

from oracle import attn_oracle as O
from xdit_amd import ops, ring, usp

pytestmark = pytest.mark.gpu


def _ring_case(seed):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(1, 128, 4, 32, generator=g).half() for _ in range(3))


@pytest.mark.parametrize("rank", [0, 1])
@pytest.mark.parametrize("strategy", ["none", "rear", "front"])
def test_ring_flash_attn_func_like_the_reference(gpu, rank, strategy):
    q, k, v = _ring_case(42)
    jq, jk, jv = _ring_case(43)
    world = 2
    if strategy == "rear":
        kk, vv = torch.cat([k, jk], 1), torch.cat([v, jv], 1)
    elif strategy == "front":
        kk, vv = torch.cat([jk, k], 1), torch.cat([jv, v], 1)
    else:
        kk, vv = k, v
    # one-shot reference on the full tensors (BSHD -> BHSD for the oracle), this rank's query rows
    ro, _ = O.attn_fwd_ref(q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2))
    ref = ro.transpose(1, 2).chunk(world, dim=1)[rank]
    local_q = q.chunk(world, dim=1)[rank].to(gpu)
    kw = {}
    if strategy != "none":
        kw = dict(joint_tensor_key=jk.to(gpu), joint_tensor_value=jv.to(gpu), joint_strategy=strategy)
    out = ring.xdit_ring_flash_attn_func(q=local_q, k=k.to(gpu), v=v.to(gpu), dropout_p=0.0, causal=False,
                                         window_size=(-1, -1), group=ring.LocalRing(world, rank), **kw)
    assert out.shape == ref.shape and out.dtype == torch.float16
    torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-3, atol=1e-3)
    # the reference's first case is causal, which this path does not implement: it must say so
    with pytest.raises(NotImplementedError):
        ring.xdit_ring_flash_attn_func(q=local_q, k=k.to(gpu), v=v.to(gpu), causal=True, group=ring.LocalRing(world, rank))


@pytest.fixture(scope="module")
def usp_case(gpu):
    g = torch.Generator().manual_seed(14867)
    q, k, v = (torch.randn(1, 24, 14867, 128, generator=g).bfloat16() for _ in range(3))
    rows = [0, 1, 383, 384, 7000, 14847, 14848, 14866]
    ro, rl = O.attn_rows_ref(q, k, v, rows)
    return dict(q=q.to(gpu), k=k.to(gpu), v=v.to(gpu), rows=rows, ro=ro, rl=rl)


def test_usp_and_ring_attn_at_the_reference_shape(gpu, usp_case):
    c = usp_case
    out = usp.USP(c["q"], c["k"], c["v"], dropout_p=0.0, is_causal=False)
    assert (out[:, :, c["rows"]].double().cpu() - c["ro"]).abs().max().item() < 0.05   # places=1
    assert (out[:, :, c["rows"]].double().cpu() - c["ro"]).abs().max().item() <= 2e-2  # this build's bar
    fn = usp._get_attention_function()
    ring_out = usp.ring_attn(fn, c["q"], c["k"], c["v"], dropout_p=0.0, is_causal=False)
    assert (ring_out.float() - out.float()).abs().max().item() < 0.05
    # S = 14867 is not divisible into ring chunks: the reference's torch ring would need padding too
    with pytest.raises(ValueError):
        usp.ring_attn(fn, c["q"], c["k"], c["v"], ring_chunks=4)
    # torch's own attention on the GPU, the reference's comparison backend, where this build has it
    try:
        torch_out = torch.nn.functional.scaled_dot_product_attention(c["q"][:, :2], c["k"][:, :2], c["v"][:, :2])
    except RuntimeError as e:  # no usable SDPA kernel for this shape on this build
        pytest.skip(f"torch SDPA unavailable: {e}")
    diff = (torch_out.float() - out[:, :2].float()).abs().max().item()
    assert diff < 0.05


def test_usp_hybrid_equivalence(gpu, usp_case):
    c = usp_case
    layer = ring.xFuserLongContextAttention()
    u = usp.USP(c["q"], c["k"], c["v"], dropout_p=0.0, is_causal=False)
    h = layer(None, c["q"].transpose(1, 2), c["k"].transpose(1, 2), c["v"].transpose(1, 2),
              dropout_p=0.0, causal=False).transpose(1, 2)
    assert (u.float() - h.float()).abs().max().item() < 5e-4  # places=3


def test_usp_hybrid_joint_equivalence(gpu, usp_case):
    c = usp_case
    g = torch.Generator().manual_seed(64)
    jq, jk, jv = (torch.randn(1, 24, 64, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
    layer = ring.xFuserLongContextAttention()
    u = usp.USP(c["q"], c["k"], c["v"], dropout_p=0.0, is_causal=False, joint_query=jq, joint_key=jk,
                joint_value=jv, joint_strategy="rear")
    h = layer(None, c["q"].transpose(1, 2), c["k"].transpose(1, 2), c["v"].transpose(1, 2), dropout_p=0.0,
              causal=False, joint_tensor_query=jq.transpose(1, 2), joint_tensor_key=jk.transpose(1, 2),
              joint_tensor_value=jv.transpose(1, 2), joint_strategy="rear").transpose(1, 2)
    assert u.shape == (1, 24, 14867 + 64, 128)
    assert (u.float() - h.float()).abs().max().item() < 5e-4  # places=3
    # and against the oracle on probe rows of the joint problem (queries: [image; joint])
    rows = [0, 14866, 14867, 14930]
    qq = torch.cat([c["q"], jq], 2).cpu()
    ro, _ = O.attn_rows_ref(qq, torch.cat([c["k"], jk], 2).cpu(), torch.cat([c["v"], jv], 2).cpu(), rows)
    assert (u[:, :, rows].double().cpu() - ro).abs().max().item() <= 2e-2
