"""Pins the CPU oracle (oracle/attn_oracle.py, oracle/attn_ref.c) WITHOUT the reference:
brute force on tiny inputs, torch's own CPU attention ops, the mathematics of the merge, the
committed golden fixtures.  Each check is chosen so that a plausible mistake (a missing scale, a
log2 instead of ln, a swapped operand in the merge, a transposed K) fails it."""
import ctypes
import math
import os
import subprocess

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")


# ------------------------------------------------------------------ attention forward
@pytest.mark.parametrize("Sq,Sk,D", [(1, 1, 4), (3, 8, 4), (8, 3, 8), (17, 17, 8), (5, 33, 8)])
def test_attn_ref_matches_bruteforce(Sq, Sk, D):
    g = torch.Generator().manual_seed(100 + Sq * 37 + Sk)
    q = torch.randn(Sq, D, generator=g, dtype=torch.float64)
    k = torch.randn(Sk, D, generator=g, dtype=torch.float64)
    v = torch.randn(Sk, D, generator=g, dtype=torch.float64)
    scale = 0.37  # deliberately not D**-0.5: a dropped scale must show
    bo, bl = O.attn_bruteforce(q.tolist(), k.tolist(), v.tolist(), scale)
    o, l = O.attn_fwd_ref(q[None, None], k[None, None], v[None, None], scale)
    assert torch.allclose(o[0, 0], torch.tensor(bo, dtype=torch.float64), atol=1e-13, rtol=1e-12)
    assert torch.allclose(l[0, 0], torch.tensor(bl, dtype=torch.float64), atol=1e-13, rtol=1e-12)


def test_tiny_golden_fixture():
    z = np.load(os.path.join(GOLD, "tiny_bruteforce.npz"))
    for n in range(5):
        q, k, v = (torch.from_numpy(z[f"t{n}_{x}"]) for x in "qkv")
        o, l = O.attn_fwd_ref(q[None, None], k[None, None], v[None, None], q.shape[-1] ** -0.5)
        assert np.allclose(o[0, 0].numpy(), z[f"t{n}_out"], atol=1e-13)
        assert np.allclose(l[0, 0].numpy(), z[f"t{n}_lse"], atol=1e-13)


def test_attn_ref_matches_torch_cpu_ops():
    """out against aten._scaled_dot_product_attention_math (the op the reference's SDPA_MATH
    backend calls) and lse against aten._scaled_dot_product_flash_attention_for_cpu."""
    g = torch.Generator().manual_seed(3)
    q = torch.randn(2, 3, 50, 16, generator=g)
    k = torch.randn(2, 3, 70, 16, generator=g)
    v = torch.randn(2, 3, 70, 16, generator=g)
    o, l = O.attn_fwd_ref(q, k, v)
    mo, attn = torch.ops.aten._scaled_dot_product_attention_math(q, k, v)
    assert attn.shape == (2, 3, 50, 70)  # second output of the math op is the S x S matrix, not lse
    assert torch.allclose(o.float(), mo, atol=2e-6)
    fo, fl = torch.ops.aten._scaled_dot_product_flash_attention_for_cpu(q, k, v)
    assert torch.allclose(o.float(), fo, atol=2e-6)
    assert torch.allclose(l.float(), fl, atol=2e-6)  # natural log, scale included
    so = O.sdpa_cpu(q, k, v)
    assert torch.allclose(o.float(), so, atol=2e-6)


def test_attn_ref_uniform_keys_closed_form():
    """All keys equal -> softmax uniform: out = mean(v), lse = s + ln(Sk)."""
    q = torch.randn(1, 1, 4, 8, dtype=torch.float64)
    k = torch.ones(1, 1, 10, 8, dtype=torch.float64) * 0.5
    v = torch.randn(1, 1, 10, 8, dtype=torch.float64)
    o, l = O.attn_fwd_ref(q, k, v, 0.25)
    assert torch.allclose(o[0, 0], v[0, 0].mean(0).expand(4, 8), atol=1e-14)
    s = 0.25 * (q[0, 0] * 0.5).sum(-1)
    assert torch.allclose(l[0, 0], s + math.log(10), atol=1e-14)


def test_attn_rows_ref_is_a_row_subset():
    q, k, v = O.make_qkv(1, 2, 64, 8, seed=5)
    o, l = O.attn_fwd_ref(q, k, v)
    ro, rl = O.attn_rows_ref(q, k, v, [0, 5, 63])
    assert torch.allclose(ro, o[:, :, [0, 5, 63]], atol=1e-14) and torch.allclose(rl, l[:, :, [0, 5, 63]], atol=1e-14)


def test_c_twin_matches_python_oracle():
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "_build", "libattn_ref.so"))
    Sq, Sk, D = 9, 21, 8
    q, k, v = (torch.randn(n, D) for n in (Sq, Sk, Sk))
    out = np.zeros((Sq, D)); lse = np.zeros(Sq)
    fp = ctypes.POINTER(ctypes.c_float); dp = ctypes.POINTER(ctypes.c_double)
    lib.attn_ref_fwd.argtypes = [fp, fp, fp, ctypes.c_long, ctypes.c_long, ctypes.c_int, ctypes.c_double, dp, dp]
    rc = lib.attn_ref_fwd(q.numpy().ctypes.data_as(fp), k.numpy().ctypes.data_as(fp), v.numpy().ctypes.data_as(fp),
                          Sq, Sk, D, 0.3, out.ctypes.data_as(dp), lse.ctypes.data_as(dp))
    assert rc == 0
    o, l = O.attn_fwd_ref(q[None, None], k[None, None], v[None, None], 0.3)
    assert np.allclose(out, o[0, 0].numpy(), atol=1e-13) and np.allclose(lse, l[0, 0].numpy(), atol=1e-13)
    # merge twin
    a = np.random.randn(6, D); al = np.random.randn(6); b = np.random.randn(6, D); bl = np.random.randn(6)
    ro, rl = O.merge_ref(torch.from_numpy(a), torch.from_numpy(al), torch.from_numpy(b), torch.from_numpy(bl))
    lib.attn_ref_merge.argtypes = [dp, dp, dp, dp, ctypes.c_long, ctypes.c_int]
    a2, al2 = a.copy(), al.copy()
    lib.attn_ref_merge(a2.ctypes.data_as(dp), al2.ctypes.data_as(dp), b.ctypes.data_as(dp), bl.ctypes.data_as(dp), 6, D)
    assert np.allclose(a2, ro.numpy(), atol=1e-14) and np.allclose(al2, rl.numpy(), atol=1e-14)


# ------------------------------------------------------------------ merge
def _rand_partials(seed, shape=(2, 3, 11), D=8):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, D, generator=g, dtype=torch.float64), torch.randn(*shape, generator=g, dtype=torch.float64) * 4,
            torch.randn(*shape, D, generator=g, dtype=torch.float64), torch.randn(*shape, generator=g, dtype=torch.float64) * 4)


def test_merge_is_logaddexp_identity():
    out, lse, bo, bl = _rand_partials(1)
    no, nl = O.merge_ref(out, lse, bo, bl)
    co, cl = O.merge_closed_form(out, lse, bo, bl)
    assert torch.allclose(no, co, atol=1e-13) and torch.allclose(nl, cl, atol=1e-13)


def test_merge_golden_fixture():
    z = np.load(os.path.join(GOLD, "merge_fold.npz"))
    no, nl = O.merge_ref(*(torch.from_numpy(z[n]) for n in ("out", "lse", "block_out", "block_lse")))
    assert np.allclose(no.numpy(), z["new_out"], atol=1e-13) and np.allclose(nl.numpy(), z["new_lse"], atol=1e-13)


def test_merge_special_cases():
    out, lse, bo, bl = _rand_partials(2)
    # a block with no mass (lse = -inf) is the identity
    no, nl = O.merge_ref(out, lse, bo, torch.full_like(bl, -math.inf))
    assert torch.equal(no, out) and torch.equal(nl, lse)
    # equal lse: arithmetic mean and lse + ln 2
    no, nl = O.merge_ref(out, lse, bo, lse.clone())
    assert torch.allclose(no, 0.5 * (out + bo), atol=1e-14) and torch.allclose(nl, lse + math.log(2), atol=1e-14)
    # commutative: swapping accumulator and block gives the same result
    a, b_ = O.merge_ref(out, lse, bo, bl)
    c, d = O.merge_ref(bo, bl, out, lse)
    assert torch.allclose(a, c, atol=1e-13) and torch.allclose(b_, d, atol=1e-13)
    # a dominant block wins
    no, nl = O.merge_ref(out, lse, bo, lse + 80.0)
    assert torch.allclose(no, bo, atol=1e-12) and torch.allclose(nl, lse + 80.0, atol=1e-12)


@pytest.mark.parametrize("P,order", [(2, None), (4, None), (4, [0, 1, 2, 3]), (3, [2, 0, 1])])
def test_fold_of_any_partition_equals_single_pass(P, order):
    q, k, v = O.make_qkv(1, 2, 48, 8, seed=9)
    o, l = O.attn_fwd_ref(q, k, v)
    ro, rl = O.ring_forward_ref(q, k, v, P, order)
    assert torch.allclose(ro, o, atol=1e-13) and torch.allclose(rl, l, atol=1e-13)


@pytest.mark.parametrize("strategy", ["front", "rear"])
def test_joint_strategy_equals_concatenated_attention(strategy):
    q, k, v = O.make_qkv(1, 2, 32, 8, seed=10)
    jq, jk, jv = O.make_qkv(1, 2, 6, 8, seed=11)
    cat = (lambda a, b: torch.cat([a, b], 2)) if strategy == "rear" else (lambda a, b: torch.cat([b, a], 2))
    qq = cat(q, jq)
    o, l = O.attn_fwd_ref(qq, cat(k, jk), cat(v, jv))
    ro, rl = O.ring_forward_ref(qq, k, v, 4, joint_k=jk, joint_v=jv, joint_strategy=strategy)
    assert torch.allclose(ro, o, atol=1e-13) and torch.allclose(rl, l, atol=1e-13)
    # key order does not matter: front and rear give the same rows
    o2, _ = O.attn_fwd_ref(qq, torch.cat([jk, k], 2), torch.cat([jv, v], 2))
    o3, _ = O.attn_fwd_ref(qq, torch.cat([k, jk], 2), torch.cat([v, jv], 2))
    assert torch.allclose(o2, o3, atol=1e-13)


def test_update_out_and_lse_ref_layout_and_first_call():
    """BSHD accumulator, lse kept as (B,S,H,1); first call copies; the epilogue
    lse.squeeze(-1).transpose(1,2) returns (B,H,S)."""
    B, S, H, D = 2, 5, 3, 4
    bo = torch.randn(B, S, H, D).bfloat16(); bl = torch.randn(B, H, S)
    out, lse = O.update_out_and_lse_ref(None, None, bo, bl)
    assert out.dtype == torch.float32 and out.shape == (B, S, H, D) and lse.shape == (B, S, H, 1)
    assert torch.equal(out, bo.float()) and torch.equal(lse.squeeze(-1).transpose(1, 2), bl)
    bo2 = torch.randn(B, S, H, D).bfloat16(); bl2 = torch.randn(B, H, S)
    out2, lse2 = O.update_out_and_lse_ref(out, lse, bo2, bl2)
    ro, rl = O.merge_ref(bo.float().transpose(1, 2), bl, bo2.float().transpose(1, 2), bl2, dtype=torch.float32)
    assert torch.allclose(out2.transpose(1, 2), ro, atol=1e-6) and torch.allclose(lse2.squeeze(-1).transpose(1, 2), rl, atol=1e-6)


# ------------------------------------------------------------------ fp8
def test_per_tensor_quant_ref_properties():
    x = torch.randn(2, 3, 16, 8) * 5
    y, d = O.per_tensor_quant_ref(x)
    assert y.dtype == torch.float8_e4m3fn and d.shape == (2, 3) and d.dtype == torch.float32
    assert torch.all(d == d[0, 0])                      # one scale for the whole tensor
    assert d[0, 0].item() == pytest.approx(x.abs().max().item() / 448.0, rel=1e-7)
    assert y.float().abs().max().item() == 448.0         # the abs-max element maps to the fp8 maximum
    # round trip error bounded by half an ulp of e4m3 (2^-4 relative) plus the subnormal step
    back = y.float() * d[0, 0]
    assert torch.all((back - x).abs() <= x.abs() * 2 ** -4 + d[0, 0] * 2 ** -10)
    # exact known answers: 448*scale -> 0x7E, scale -> 0x38 (1.0), 0 -> 0x00, -scale*2 -> 0xC0
    s = torch.tensor(0.5)
    yy, _ = O.per_tensor_quant_ref(torch.tensor([[[[224.0, 0.5, 0.0, -1.0]]]]), scale=s)
    assert yy.view(torch.uint8).flatten().tolist() == [0x7E, 0x38, 0x00, 0xC0]


def test_per_head_quant_ref_properties():
    x = torch.randn(2, 3, 16, 8) * torch.arange(1, 7).reshape(2, 3, 1, 1)
    y, d = O.per_head_quant_ref(x)
    assert torch.allclose(d, x.abs().amax((2, 3)) / 448.0, rtol=1e-7)
    assert torch.all(y.float().abs().amax((2, 3)) == 448.0)
    y0, d0 = O.per_head_quant_ref(torch.zeros(1, 1, 4, 8))
    assert d0.item() == 1.0 and torch.all(y0.float() == 0)


# ------------------------------------------------------------------ configurations
def test_config_generators_are_seeded_and_shaped():
    a = O.make_config("c2_flux1024", S=256)
    b = O.make_config("c2_flux1024", S=256)
    assert a["q"].dtype == torch.bfloat16 and a["q"].shape == (1, 24, 256, 128)
    assert all(torch.equal(a[n], b[n]) for n in "qkv")
    # RMSNorm'd q/k: per-row RMS within the gain range
    rms = a["q"].float().pow(2).mean(-1).sqrt()
    assert 0.75 < rms.min() and rms.max() < 1.25
    c = O.make_config("c5_wan720p_shard_fp8", S=128)
    assert c["q"].dtype == torch.float8_e4m3fn and c["q_descale"].shape == (1, 5)
    z = np.load(os.path.join(GOLD, "c5_fp8_s2048_rows.npz"))
    c2048 = O.make_config("c5_wan720p_shard_fp8", S=2048)
    assert np.array_equal(c2048["q"].view(torch.uint8)[0, 0, 0].numpy(), z["q_bytes_head0_row0"])
    assert np.array_equal(c2048["k_descale"].numpy(), z["k_descale"])


def test_c1_golden_fixture_against_oracle_and_torch():
    z = np.load(os.path.join(GOLD, "c1_pixart512.npz"))
    c1 = O.make_config("c1_pixart512")
    o, l = O.attn_fwd_ref(c1["q"], c1["k"], c1["v"], 72 ** -0.5)
    assert np.allclose(o[:, :, ::37].numpy(), z["out_rows"], atol=1e-6)
    assert np.allclose(l.numpy(), z["lse"], atol=1e-6)
    mo, _ = torch.ops.aten._scaled_dot_product_attention_math(c1["q"], c1["k"], c1["v"])
    assert np.allclose(mo[:, :, ::37].numpy(), z["out_rows"], atol=5e-6)


# ---------------------------------------------------------------------------- Hadamard rotation
@pytest.mark.parametrize("n", [1, 2, 8, 32, 128])
def test_hadamard_matrix_sign_rule_and_orthonormality(n):
    """Sylvester's matrix has entries (-1)^popcount(i & j); scaled by 1/sqrt(n) it is symmetric
    and orthonormal.  A transposed block or a wrong sign in the recursion fails the sign rule."""
    R = O.hadamard_matrix(n)
    i = torch.arange(n)
    pop = torch.tensor([[bin(int(a) & int(b)).count("1") for b in i] for a in i])
    expect = torch.where(pop % 2 == 0, 1.0, -1.0).double() * float(torch.tensor(1.0) / torch.tensor(n ** 0.5))
    assert torch.allclose(R, expect, atol=1e-7)
    assert torch.allclose(R @ R.T, torch.eye(n, dtype=torch.float64), atol=1e-6)
    assert torch.equal(R, R.T)


def _fwht(x):
    """Textbook in-place fast Walsh-Hadamard transform (natural order), pure Python."""
    x = list(x)
    h = 1
    while h < len(x):
        for i in range(0, len(x), 2 * h):
            for j in range(i, i + h):
                x[j], x[j + h] = x[j] + x[j + h], x[j] - x[j + h]
        h *= 2
    return x


@pytest.mark.parametrize("block", [8, 32, 128])
def test_hadamard_rotate_ref_against_fwht_and_invariance(block):
    g = torch.Generator().manual_seed(block)
    x = torch.randn(1, 2, 5, 128, generator=g, dtype=torch.float64)
    y = O.hadamard_rotate_ref(x, block)
    r = float(torch.tensor(1.0) / torch.tensor(block ** 0.5))  # the fp32 normalisation the reference applies
    for row in (0, 3):
        for b0 in range(0, 128, block):
            ref = [v * r for v in _fwht(x[0, 1, row, b0:b0 + block].tolist())]
            assert torch.allclose(y[0, 1, row, b0:b0 + block], torch.tensor(ref, dtype=torch.float64), atol=1e-12)
    # rotating q and k alike leaves the logits unchanged (up to the fp32 rounding of 1/sqrt(n))
    k = torch.randn(1, 2, 7, 128, generator=g, dtype=torch.float64)
    s0 = x @ k.transpose(-1, -2)
    s1 = y @ O.hadamard_rotate_ref(k, block).transpose(-1, -2)
    assert torch.allclose(s0, s1, rtol=1e-6, atol=1e-6)
    # bf16: result is the correctly rounded product with the matrix held in bf16
    xb = x.to(torch.bfloat16)
    yb = O.hadamard_rotate_ref(xb, block)
    assert yb.dtype == torch.bfloat16
    Rb = O.hadamard_matrix(block, torch.bfloat16).double()
    blk = xb.double()[..., :block] @ Rb
    assert torch.equal(yb[..., :block], blk.to(torch.bfloat16))
    # an outlier is spread evenly over its block
    e = torch.zeros(1, 1, 1, 128, dtype=torch.float64)
    e[..., 5] = 64.0
    ye = O.hadamard_rotate_ref(e, block)
    assert torch.allclose(ye[..., :block].abs(), torch.full((block,), 64.0 * r, dtype=torch.float64))
    assert (ye[..., block:] == 0).all() or block == 128


# ---------------------------------------------------------------------------- prologue
def test_rms_norm_ref_against_torch_rms_norm_and_roundings():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 7, 3, 128, generator=g) * 3
    w = 0.8 + 0.4 * torch.rand(128, generator=g)
    # float64 inputs: no rounding anywhere except the fp32 statistic -> torch's own rms_norm
    ref = F.rms_norm(x.double(), (128,), w.double(), 1e-6)
    got = O.rms_norm_ref(x.double(), w.double(), 1e-6)
    assert torch.allclose(got, ref, rtol=1e-6, atol=1e-7)
    # a dropped eps or a mean over the wrong axis fails this
    tiny = torch.full((1, 1, 1, 128), 1e-4)
    assert torch.allclose(O.rms_norm_ref(tiny, None, 1e-6), tiny / (1e-8 + 1e-6) ** 0.5, rtol=1e-5)
    # bf16: result = bf16(bf16(x * rs) * w), i.e. two roundings, and never further than 2 ulp from exact
    xb, wb = x.bfloat16(), w.bfloat16()
    got = O.rms_norm_ref(xb, wb, 1e-6)
    assert got.dtype == torch.bfloat16
    rs = torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-6)
    two = ((xb.float() * rs).bfloat16().float() * wb.float()).bfloat16()
    assert torch.equal(got, two)
    exact = F.rms_norm(xb.double(), (128,), wb.double(), 1e-6)
    assert ((got.double() - exact).abs() <= 2.0 ** -7 * exact.abs() + 1e-30).all()
    assert O.rms_norm_ref(xb, None, 1e-6).dtype == torch.bfloat16


@pytest.mark.parametrize("sequence_dim", [1, 2])
def test_apply_rotary_emb_ref_is_complex_multiplication(sequence_dim):
    g = torch.Generator().manual_seed(6)
    S, D = 9, 16
    x = torch.randn(2, 3, S, D, generator=g, dtype=torch.float64)
    ang = torch.randn(S, D // 2, generator=g, dtype=torch.float64)
    xin = x if sequence_dim == 2 else x.transpose(1, 2)
    # interleaved pairs (2i, 2i+1) as complex numbers times e^{i angle}
    cos, sin = ang.cos().repeat_interleave(2, 1), ang.sin().repeat_interleave(2, 1)
    got = O.apply_rotary_emb_ref(xin, (cos, sin), -1, sequence_dim)
    got = got if sequence_dim == 2 else got.transpose(1, 2)
    z = torch.view_as_complex(x.reshape(2, 3, S, D // 2, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(got, torch.view_as_real(z).flatten(3), atol=1e-12)
    # pairs (j, j + D/2)
    cos2, sin2 = torch.cat([ang.cos()] * 2, 1), torch.cat([ang.sin()] * 2, 1)
    got2 = O.apply_rotary_emb_ref(xin, (cos2, sin2), -2, sequence_dim)
    got2 = got2 if sequence_dim == 2 else got2.transpose(1, 2)
    z2 = torch.complex(x[..., :D // 2], x[..., D // 2:]) * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(got2, torch.cat([z2.real, z2.imag], -1), atol=1e-12)
    # a rotation preserves the length of every pair; angle 0 is the identity
    assert torch.allclose(got.reshape(2, 3, S, -1, 2).norm(dim=-1), x.reshape(2, 3, S, -1, 2).norm(dim=-1), atol=1e-12)
    one, zero = torch.ones(S, D, dtype=torch.float64), torch.zeros(S, D, dtype=torch.float64)
    assert torch.equal(O.apply_rotary_emb_ref(xin.float(), (one.float(), zero.float()), -1, sequence_dim), xin.float())
    # the Wan form reads cos[2i] and sin[2i+1] for a pair: same result on pair-repeated tables
    wan = O.apply_rotary_emb_wan_ref(x.transpose(1, 2), cos[None, :, None, :], sin[None, :, None, :])
    assert torch.allclose(wan.transpose(1, 2), got, atol=1e-12)


def test_rope_tables_shape_and_pairing():
    cos, sin = O.rope_tables(11, 128, seed=1)
    assert cos.shape == (11, 128) and cos.dtype == torch.float32
    assert torch.equal(cos[:, 0::2], cos[:, 1::2]) and torch.equal(sin[:, 0::2], sin[:, 1::2])
    assert torch.allclose(cos * cos + sin * sin, torch.ones(11, 128), atol=1e-6)
    cos, sin = O.rope_tables(11, 64, seed=1, axes=(), interleave=False)
    assert torch.equal(cos[:, :32], cos[:, 32:])
