"""GPU parity of the fused pre-attention prologue (RMSNorm + rotary embedding + re-layout) against
the CPU oracle's restatement of the processors' steps.

Bars: the rotation and the re-layout are bit-exact (same fp32 products and sums, one rounding).
The norm's statistic is a sum of D squares whose order differs between the kernel and torch's CPU
reduction, so a normalised value may land on the other side of a rounding boundary: at least
99.5 % of the elements must be bit-equal and the rest within one unit in the last place of the
dtype (2^-7 relative for bf16, 2^-10 for fp16); fp32 results within 2^-21 relative.
"""
import pytest
import torch

from oracle import attn_oracle as O
from xdit_amd import ops, prologue

pytestmark = pytest.mark.gpu
ULP = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -21}


def _close(got, ref, dtype, exact=False):
    got, ref = got.detach().cpu(), ref.detach().cpu()
    assert got.shape == ref.shape and got.dtype == ref.dtype
    if exact:
        assert torch.equal(got, ref)
        return
    if dtype != torch.float32:  # fp32 results carry the summation order in their last bits
        same = (got == ref).float().mean().item()
        assert same >= 0.995, same
    d = (got.double() - ref.double()).abs()
    assert (d <= ULP[dtype] * ref.double().abs() + 1e-30).all(), d.max().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,S,H,D", [(1, 77, 3, 128), (2, 5, 24, 128), (1, 130, 2, 64), (1, 33, 5, 72), (1, 9, 1, 256)])
def test_head_norm_vs_oracle(gpu, dtype, B, S, H, D):
    g = torch.Generator().manual_seed(S * H + D)
    x = (torch.randn(B, S, H, D, generator=g) * 2).to(dtype)
    w = (0.8 + 0.4 * torch.rand(D, generator=g)).to(dtype)
    ref = O.rms_norm_ref(x, w, 1e-6)
    # BSHD in -> BHSD-contiguous out
    y = ops.qk_prologue(x.to(gpu).transpose(1, 2), weight=w.to(gpu), eps=1e-6, norm="head")
    assert y.is_contiguous() and y.shape == (B, H, S, D)
    _close(y, ref.transpose(1, 2).contiguous(), dtype)
    # no gain, module form, any leading shape
    m = prologue.RMSNorm(D, eps=1e-5, elementwise_affine=False)
    _close(m(x.to(gpu)), O.rms_norm_ref(x, None, 1e-5), dtype)
    m = prologue.RMSNorm(D, eps=1e-6, device=gpu, dtype=dtype)
    with torch.no_grad():
        m.weight.copy_(w)
    _close(m(x.to(gpu)[0]), ref[0], dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("unbind,D", [(-1, 128), (-2, 128), (-1, 72), (-2, 64), (-1, 8)])
@pytest.mark.parametrize("sequence_dim", [1, 2])
def test_apply_rotary_emb_bit_exact(gpu, dtype, unbind, D, sequence_dim):
    g = torch.Generator().manual_seed(D + unbind)
    B, H, S = 2, 3, 70
    x = torch.randn((B, S, H, D) if sequence_dim == 1 else (B, H, S, D), generator=g).to(dtype)
    cos, sin = O.rope_tables(S, D, seed=D, axes=(), interleave=(unbind == -1))
    ref = O.apply_rotary_emb_ref(x, (cos, sin), unbind, sequence_dim)
    got = prologue.apply_rotary_emb(x.to(gpu), (cos.to(gpu), sin.to(gpu)), use_real_unbind_dim=unbind, sequence_dim=sequence_dim)
    _close(got, ref, dtype, exact=True)
    # tables that are NOT pair-repeated: every element uses its own cos / sin entry
    cos2, sin2 = torch.randn(S, D, generator=g), torch.randn(S, D, generator=g)
    ref = O.apply_rotary_emb_ref(x, (cos2, sin2), unbind, sequence_dim)
    got = prologue.apply_rotary_emb(x.to(gpu), (cos2.to(gpu), sin2.to(gpu)), use_real_unbind_dim=unbind, sequence_dim=sequence_dim)
    _close(got, ref, dtype, exact=True)


def test_wan_rotation_and_token_norm(gpu):
    """Wan: RMSNorm over the un-split projection (all heads of a token, H*D gains), then the
    model's own rotation formula (transformer_wan.py:99-122)."""
    g = torch.Generator().manual_seed(3)
    B, S, H, D = 1, 50, 40, 128
    x = torch.randn(B, S, H * D, generator=g).bfloat16()
    w = (0.8 + 0.4 * torch.rand(H * D, generator=g)).bfloat16()
    cos, sin = O.rope_tables(S, D, seed=2, axes=(44, 42, 42))
    cos4, sin4 = cos[None, :, None, :], sin[None, :, None, :]
    normed = O.rms_norm_ref(x, w, 1e-6).unflatten(2, (H, D))
    ref = O.apply_rotary_emb_wan_ref(normed, cos4, sin4)
    # rotation alone: bit-exact, and on tables that are not pair-repeated too
    got = prologue.apply_rotary_emb_wan(normed.to(gpu), cos4.to(gpu), sin4.to(gpu))
    _close(got, ref, torch.bfloat16, exact=True)
    c2, s2 = torch.randn(1, S, 1, D, generator=g), torch.randn(1, S, 1, D, generator=g)
    _close(prologue.apply_rotary_emb_wan(normed.to(gpu), c2.to(gpu), s2.to(gpu)),
           O.apply_rotary_emb_wan_ref(normed, c2, s2), torch.bfloat16, exact=True)
    # fused: token-wide norm + rotation + BHSD
    y = prologue.norm_rope(x.to(gpu).unflatten(2, (H, D)), weight=w.to(gpu), freqs_cis=(cos.to(gpu), sin.to(gpu)),
                           sequence_dim=1, norm="token", rope="wan")
    assert y.shape == (B, H, S, D) and y.is_contiguous()
    got, want = y.cpu(), ref.transpose(1, 2)
    # a normalised value that differs by one rounding step is then rotated with its partner
    assert (got == want).float().mean().item() >= 0.99
    assert (got.double() - want.double()).abs().max().item() <= 2.0 ** -6 * want.double().abs().max().item()
    with pytest.raises(NotImplementedError):
        ops.qk_prologue(torch.zeros(1, 80, 4, 128, device=gpu), norm="token")  # H*D above the limit


def test_hunyuan_video_partial_rotation(gpu):
    """HunyuanVideo (transformer_hunyuan_video.py:48-83): BHSD input, per-head norm, rotation of
    the video rows only; the text rows behind them pass through normalised."""
    g = torch.Generator().manual_seed(4)
    B, H, S, T, D = 1, 3, 200, 24, 128
    x = torch.randn(B, H, S, D, generator=g).bfloat16()
    w = (0.8 + 0.4 * torch.rand(D, generator=g)).bfloat16()
    cos, sin = O.rope_tables(S - T, D, seed=8)
    n = O.rms_norm_ref(x, w, 1e-6)
    ref = torch.cat([O.apply_rotary_emb_ref(n[:, :, :-T], (cos, sin)), n[:, :, -T:]], dim=2)
    y = prologue.norm_rope(x.to(gpu), weight=w.to(gpu), freqs_cis=(cos.to(gpu), sin.to(gpu)), sequence_dim=2,
                           rope_rows=S - T)
    got = y.cpu()
    assert (got == ref).float().mean().item() >= 0.99
    assert (got.double() - ref.double()).abs().max().item() <= 2.0 ** -6 * ref.double().abs().max().item()
    # rows offset the other way (CogVideoX rotates the rows AFTER the text rows)
    ref2 = torch.cat([n[:, :, :T], O.apply_rotary_emb_ref(n[:, :, T:], (cos, sin))], dim=2)
    y2 = ops.qk_prologue(x.to(gpu), weight=w.to(gpu), norm="head", rotary_emb=(cos.to(gpu), sin.to(gpu)), rope_row0=T)
    assert (y2.cpu() == ref2).float().mean().item() >= 0.99
    _close(y2[:, :, :T], n[:, :, :T], torch.bfloat16)


def test_flux_joint_qkv_equals_processor_steps_and_feeds_attention(gpu):
    """Lines 116-147 + 170-172 of the Flux processor restated with the oracle's pieces, against
    the six fused launches; then attention on the fused tensors against the oracle."""
    g = torch.Generator().manual_seed(9)
    B, H, D, S_txt, S_img = 1, 4, 128, 40, 216
    mk = lambda s: torch.randn(B, s, H * D, generator=g).bfloat16()
    q, k, v, eq, ek, ev = mk(S_img), mk(S_img), mk(S_img), mk(S_txt), mk(S_txt), mk(S_txt)
    ws = [(0.8 + 0.4 * torch.rand(D, generator=g)).bfloat16() for _ in range(4)]
    cos, sin = O.rope_tables(S_txt + S_img, D, seed=5)
    hs = lambda t: t.unflatten(-1, (H, D))
    rq = torch.cat([O.rms_norm_ref(hs(eq), ws[2]), O.rms_norm_ref(hs(q), ws[0])], dim=1)
    rk = torch.cat([O.rms_norm_ref(hs(ek), ws[3]), O.rms_norm_ref(hs(k), ws[1])], dim=1)
    rv = torch.cat([hs(ev), hs(v)], dim=1)
    rq = O.apply_rotary_emb_ref(rq, (cos, sin), sequence_dim=1).transpose(1, 2)
    rk = O.apply_rotary_emb_ref(rk, (cos, sin), sequence_dim=1).transpose(1, 2)
    rv = rv.transpose(1, 2)
    d = lambda t: t.to(gpu)
    fq, fk, fv = prologue.flux_joint_qkv(d(q), d(k), d(v), d(eq), d(ek), d(ev), H, d(ws[0]), d(ws[1]), d(ws[2]), d(ws[3]),
                                         (d(cos), d(sin)))
    for t in (fq, fk, fv):
        assert t.shape == (B, H, S_txt + S_img, D) and t.is_contiguous()
    assert torch.equal(fv.cpu(), rv)
    for got, ref in ((fq, rq), (fk, rk)):
        assert (got.cpu() == ref).float().mean().item() >= 0.99
        assert (got.cpu().double() - ref.double()).abs().max().item() <= 2.0 ** -6 * ref.double().abs().max().item()
    o, l = ops.attn_fwd(fq, fk, fv)
    ro, rl = O.attn_fwd_ref(rq, rk, rv)
    assert (o.double().cpu() - ro).abs().max().item() <= 2e-2 and (l.double().cpu() - rl).abs().max().item() <= 2e-3
    # a second call of the same signature goes through the kept argument structs (pointers patched):
    # other tensors, other gains, the text and image inputs swapped in value but not in shape
    q2, k2, v2, eq2, ek2, ev2 = mk(S_img), mk(S_img), mk(S_img), mk(S_txt), mk(S_txt), mk(S_txt)
    ws2 = [(0.8 + 0.4 * torch.rand(D, generator=g)).bfloat16() for _ in range(4)]
    cos2, sin2 = O.rope_tables(S_txt + S_img, D, seed=6)
    gq, gk, gv = prologue.flux_joint_qkv(d(q2), d(k2), d(v2), d(eq2), d(ek2), d(ev2), H, d(ws2[0]), d(ws2[1]), d(ws2[2]), d(ws2[3]),
                                         (d(cos2), d(sin2)))
    assert torch.equal(gv.cpu(), torch.cat([hs(ev2), hs(v2)], dim=1).transpose(1, 2))
    sq = torch.cat([O.rms_norm_ref(hs(eq2), ws2[2]), O.rms_norm_ref(hs(q2), ws2[0])], dim=1)
    sq = O.apply_rotary_emb_ref(sq, (cos2, sin2), sequence_dim=1).transpose(1, 2)
    sk = torch.cat([O.rms_norm_ref(hs(ek2), ws2[3]), O.rms_norm_ref(hs(k2), ws2[1])], dim=1)
    sk = O.apply_rotary_emb_ref(sk, (cos2, sin2), sequence_dim=1).transpose(1, 2)
    for got, ref in ((gq, sq), (gk, sk)):
        assert (got.cpu() == ref).float().mean().item() >= 0.99
        assert (got.cpu().double() - ref.double()).abs().max().item() <= 2.0 ** -6 * ref.double().abs().max().item()
    assert torch.equal(fv.cpu(), rv)   # the first call's outputs were not touched


def test_batch_equals_single_launches(gpu):
    """One launch of several jobs gives the bits of the separate launches."""
    g = torch.Generator().manual_seed(11)
    xs = [torch.randn(1, s, 6, 128, generator=g).bfloat16().to(gpu) for s in (40, 300, 7)]
    w = (0.8 + 0.4 * torch.rand(128, generator=g)).bfloat16().to(gpu)
    cos, sin = (t.to(gpu) for t in O.rope_tables(300, 128, seed=3))
    jobs = [dict(x=xs[0].transpose(1, 2), weight=w, norm="head", rotary_emb=(cos[:40], sin[:40])),
            dict(x=xs[1].transpose(1, 2), weight=w, norm="head", rotary_emb=(cos, sin), rope="wan"),
            dict(x=xs[2].transpose(1, 2))]
    got = ops.qk_prologue_batch(jobs)
    for j, o in zip(jobs, got):
        assert torch.equal(o, ops.qk_prologue(**j))
    with pytest.raises(ValueError):
        ops.qk_prologue_batch([])
    with pytest.raises(ValueError):
        ops.qk_prologue_batch([dict(x=xs[0].transpose(1, 2)), dict(x=xs[1].transpose(1, 2).half())])
    with pytest.raises(NotImplementedError):
        ops.qk_prologue_batch([dict(x=xs[0].transpose(1, 2), norm="token")])


def test_relayout_only_and_argument_checks(gpu):
    x = torch.randn(2, 50, 6, 64, device=gpu).half()
    y = ops.qk_prologue(x.transpose(1, 2))
    assert y.is_contiguous() and torch.equal(y, x.transpose(1, 2))
    out = torch.zeros(2, 6, 80, 64, device=gpu).half()
    ops.qk_prologue(x.transpose(1, 2), out=out[:, :, 30:])
    assert torch.equal(out[:, :, 30:], x.transpose(1, 2)) and (out[:, :, :30] == 0).all()
    cos = torch.ones(50, 64, device=gpu)
    with pytest.raises(ValueError):
        ops.qk_prologue(x.transpose(1, 2), rotary_emb=(cos, cos), rope_rows=60)
    with pytest.raises(ValueError):
        ops.qk_prologue(x.transpose(1, 2), weight=torch.ones(32, device=gpu).half(), norm="head")
    with pytest.raises(ValueError):
        ops.qk_prologue(x.transpose(1, 2), rotary_emb=(cos.half(), cos.half()))
    with pytest.raises(NotImplementedError):
        ops.qk_prologue(torch.zeros(1, 2, 4, 72, device=gpu), rotary_emb=(torch.ones(4, 72, device=gpu),) * 2, rope="split_half")
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.qk_prologue(torch.zeros(1, 2, 4, 64))


def test_norm_rope_custom_op(gpu):
    from xdit_amd import custom_ops  # noqa: F401
    g = torch.Generator().manual_seed(21)
    x = torch.randn(1, 60, 4, 128, generator=g).bfloat16().to(gpu).transpose(1, 2)
    w = (0.8 + 0.4 * torch.rand(128, generator=g)).bfloat16().to(gpu)
    cos, sin = (t.to(gpu) for t in O.rope_tables(60, 128, seed=2))
    args = (x, w, cos, sin, 1e-6, "head", "interleaved", 0, 60)
    torch.library.opcheck(torch.ops.xdit_amd.norm_rope.default, args,
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
    eager = ops.qk_prologue(x, weight=w, norm="head", rotary_emb=(cos, sin))
    assert torch.equal(torch.ops.xdit_amd.norm_rope(*args), eager)
    fn = torch.compile(lambda a: torch.ops.xdit_amd.norm_rope(a * 1, w, cos, sin, 1e-6, "head", "interleaved", 0, 60) + 0,
                       backend="aot_eager", fullgraph=True)
    assert torch.equal(fn(x), eager)
    plain = torch.ops.xdit_amd.norm_rope(x, w, cos, sin, 0.0, "none", "none", 0, 0)
    assert torch.equal(plain, x.contiguous())
