"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs,
against the committed golden fixtures, and — at the full benchmark sizes — through
size-independent properties (fold of KV chunks == single pass, key-order invariance, layout
invariance, run-to-run determinism) plus probe rows evaluated by the oracle against the full K/V.

Tolerances (max abs error against the float64 oracle):
  bf16 / fp16 inputs   out <= 2e-2, lse <= 1e-3
  fp8 inputs           out <= 6e-2 (reference = attention of the dequantised inputs), lse <= 1e-3
  fp32 inputs          out <= 2e-5, lse <= 2e-5
"""
import os

import numpy as np
import pytest
import torch

from oracle import attn_oracle as O
from xdit_amd import attention_backend as AB
from xdit_amd import ops, ring, usp

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("sharing_mode")]
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = {torch.bfloat16: (2e-2, 1e-3), torch.float16: (2e-2, 1e-3), torch.float32: (2e-5, 2e-5)}


def _err(a, b):
    return (a.detach().double().cpu() - b.double()).abs().max().item()


def _same(a, b, mode):
    """Two runs of one call: bit-identical by default.  Under streamed sharing the KV
    iterations of a shared query tile may be grouped into its partial results differently from
    run to run; the partial results are rounded to the output type before they are folded, so
    outputs of shared tiles then differ by about one unit in the last place of the LARGEST
    values (a partial's rounding error is relative to the partial, not to the folded sum)."""
    if mode == "deterministic" or not a.is_floating_point():
        return torch.equal(a, b)
    if a.shape != b.shape:
        return False
    a, b = a.float(), b.float()
    return (a - b).abs().max().item() <= 2.0 ** -7 * max(a.abs().max().item(), 1e-30)


def _layout(t, layout, dev):
    """Put a CPU BHSD tensor on the device either BHSD-contiguous or as a BSHD-contiguous tensor
    viewed as BHSD (the two physical layouts xDiT's callers produce)."""
    if layout == "bhsd":
        return t.to(dev).contiguous()
    return t.transpose(1, 2).contiguous().to(dev).transpose(1, 2)


CASES = [
    # B, H, Sq, Sk, D
    (1, 1, 1, 1, 128), (1, 2, 5, 63, 128), (1, 2, 128, 64, 128), (1, 2, 129, 65, 128), (2, 3, 200, 333, 128),
    (1, 2, 256, 640, 128), (1, 3, 77, 1, 128), (1, 1, 1000, 127, 128), (1, 2, 300, 500, 64), (2, 2, 31, 129, 64),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
@pytest.mark.parametrize("B,H,Sq,Sk,D", CASES)
def test_attn_16bit_small_vs_oracle(gpu, dtype, layout, B, H, Sq, Sk, D):
    g = torch.Generator().manual_seed(B * 1000 + Sq * 7 + Sk)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    k = torch.randn(B, H, Sk, D, generator=g).to(dtype)
    v = torch.randn(B, H, Sk, D, generator=g).to(dtype)
    scale = 0.11 if Sq % 2 else D ** -0.5
    ro, rl = O.attn_fwd_ref(q, k, v, scale)
    o, l = ops.attn_fwd(_layout(q, layout, gpu), _layout(k, layout, gpu), _layout(v, layout, gpu), softmax_scale=scale)
    assert o.dtype == dtype and l.dtype == torch.float32 and l.shape == (B, H, Sq)
    assert _err(o, ro) <= TOL[dtype][0] and _err(l, rl) <= TOL[dtype][1]


@pytest.mark.parametrize("dtype,D", [(torch.float32, 72), (torch.float32, 8), (torch.float32, 128), (torch.float32, 64),
                                      (torch.bfloat16, 72), (torch.float16, 40), (torch.bfloat16, 96)])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (33, 31), (130, 200), (128, 32)])
def test_attn_generic_path_vs_oracle(gpu, dtype, D, Sq, Sk):
    """fp32 inputs run on the fp32 matrix cores at any head_dim; the 16-bit cases here take the
    16-bit kernel built for the next head_dim up (64 or 128)."""
    g = torch.Generator().manual_seed(D * 100 + Sq)
    q = torch.randn(2, 2, Sq, D, generator=g).to(dtype)
    k = torch.randn(2, 2, Sk, D, generator=g).to(dtype)
    v = torch.randn(2, 2, Sk, D, generator=g).to(dtype)
    ro, rl = O.attn_fwd_ref(q, k, v)
    o, l = ops.attn_fwd(_layout(q, "bshd", gpu), k.to(gpu), v.to(gpu))
    assert _err(o, ro) <= TOL[dtype][0] and _err(l, rl) <= TOL[dtype][1]


@pytest.mark.parametrize("cus", [1, 0])
@pytest.mark.parametrize("D", [72, 8, 128, 40])
@pytest.mark.parametrize("Sq,Sk,Sk2", [(1, 1, 0), (70, 33, 0), (130, 200, 45), (64, 32, 1), (257, 64, 65), (200, 31, 100)])
def test_attn_fp32_both_workgroup_forms_vs_oracle(gpu, monkeypatch, cus, D, Sq, Sk, Sk2):
    """The fp32 kernel in both forms: planned for one compute unit these problems keep 128-row
    workgroups with 32-key tiles; planned for the device's own count they are small enough to take
    64-row workgroups whose wavefront pairs split 64-key tiles and fold through LDS (key halves
    that are empty or ragged included), with and without a second KV segment."""
    monkeypatch.setitem(ops.TUNING, "cu_count", cus)
    g = torch.Generator().manual_seed(D * 1000 + Sq + Sk2)
    q = torch.randn(1, 3, Sq, D, generator=g)
    k, v = torch.randn(1, 3, Sk, D, generator=g), torch.randn(1, 3, Sk, D, generator=g)
    kw = {}
    kall, vall = k, v
    if Sk2:
        k2, v2 = torch.randn(1, 3, Sk2, D, generator=g), torch.randn(1, 3, Sk2, D, generator=g)
        kall, vall = torch.cat([k, k2], 2), torch.cat([v, v2], 2)
        kw = dict(k2=_layout(k2, "bshd", gpu), v2=v2.to(gpu))
    ro, rl = O.attn_fwd_ref(q, kall, vall)
    o, l = ops.attn_fwd(q.to(gpu), _layout(k, "bshd", gpu), v.to(gpu), **kw)
    assert _err(o, ro) <= 2e-5 and _err(l, rl) <= 2e-5


def test_tiny_bruteforce_golden(gpu):
    z = np.load(os.path.join(GOLD, "tiny_bruteforce.npz"))
    for n in (2, 3, 4):  # the head_dim 8 cases
        q, k, v = (torch.from_numpy(z[f"t{n}_{x}"]).float()[None, None] for x in "qkv")
        o, l = ops.attn_fwd(q.to(gpu), k.to(gpu), v.to(gpu))
        assert _err(o[0, 0], torch.from_numpy(z[f"t{n}_out"])) <= 2e-6
        assert _err(l[0, 0], torch.from_numpy(z[f"t{n}_lse"])) <= 2e-6


@pytest.mark.parametrize("Sk,Sk2", [(192, 70), (100, 64), (64, 1), (1, 300)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_two_kv_segments_equal_concatenation(gpu, dtype, Sk, Sk2):
    g = torch.Generator().manual_seed(Sk + Sk2)
    D = 128
    q = torch.randn(1, 2, 150, D, generator=g).to(dtype)
    k, v = (torch.randn(1, 2, Sk, D, generator=g).to(dtype) for _ in range(2))
    k2, v2 = (torch.randn(1, 2, Sk2, D, generator=g).to(dtype) for _ in range(2))
    ro, rl = O.attn_fwd_ref(q, torch.cat([k, k2], 2), torch.cat([v, v2], 2))
    o, l = ops.attn_fwd(q.to(gpu), k.to(gpu), v.to(gpu), k2=_layout(k2, "bshd", gpu), v2=_layout(v2, "bshd", gpu))
    assert _err(o, ro) <= TOL[dtype][0] and _err(l, rl) <= TOL[dtype][1]


@pytest.mark.parametrize("B,H,Sq,Sk,Sk2", [
    (1, 1, 1280, 8192, 0),     # 10 query tiles on an empty chip: every tile's KV range is cut into many parts
    (1, 3, 128, 6528, 0),      # 102 KV tiles, ranges of 4: a workgroup's range straddles two query tiles
    (1, 2, 300, 4000, 100),    # partial last KV tile, second KV segment, partial last query tile
    (2, 2, 200, 3333, 0),
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_balanced_launch_vs_oracle(gpu, sharing_mode, dtype, B, H, Sq, Sk, Sk2):
    """Problems whose query tiles do not fill the chip: the KV range of the tiles is shared between
    workgroups and folded by the combine kernel.  Must match the oracle and the plain launch."""
    g = torch.Generator().manual_seed(Sq + Sk)
    q = torch.randn(B, H, Sq, 128, generator=g).to(dtype)
    k, v = (torch.randn(B, H, Sk, 128, generator=g).to(dtype) for _ in range(2))
    k2 = v2 = None
    kk, vv = k, v
    if Sk2:
        k2, v2 = (torch.randn(B, H, Sk2, 128, generator=g).to(dtype) for _ in range(2))
        kk, vv = torch.cat([k, k2], 2), torch.cat([v, v2], 2)
    ro, rl = O.attn_fwd_ref(q, kk, vv)
    dev = lambda t: None if t is None else t.to(gpu)
    assert ops._lib.lib().xdit_attn_abi_version() >= 2
    o, l = ops.attn_fwd(dev(q), dev(k), dev(v), k2=dev(k2), v2=dev(v2))
    o1, l1 = ops.attn_fwd(dev(q), dev(k), dev(v), k2=dev(k2), v2=dev(v2), balance=False)
    assert _err(o, ro) <= TOL[dtype][0] and _err(l, rl) <= TOL[dtype][1]
    assert _err(o1, ro) <= TOL[dtype][0] and _err(l1, rl) <= TOL[dtype][1]
    assert _err(o, o1.cpu()) <= 1e-2 and _err(l, l1.cpu()) <= 1e-5
    # the workspace is scratch: a second call gives the same bits (the same values to rounding under streamed sharing)
    o2, l2 = ops.attn_fwd(dev(q), dev(k), dev(v), k2=dev(k2), v2=dev(v2))
    assert _same(o, o2, sharing_mode) and (l - l2).abs().max().item() <= (0 if sharing_mode == "deterministic" else 1e-5)


@pytest.mark.parametrize("cus", [252, 250, 100, 7])
@pytest.mark.parametrize("kind", ["bf16", "fp8"])
def test_balanced_launch_planned_for_other_compute_unit_counts(gpu, monkeypatch, kind, cus):
    """A launch planned for a compute-unit count that is not a multiple of 8 (the cu_count field of
    xdit_attn_args; such a count is what a partitioned or partly disabled GPU reports): the whole
    query tiles must still be covered exactly once.  Three rounds of whole tiles plus a sixteenth
    of a round of shared ones; at 250 units that is 1500 whole tiles, not a multiple of 8, and an
    XCD-order map that assumes one leaves tiles uncomputed."""
    monkeypatch.setitem(ops.TUNING, "cu_count", cus)
    monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", 128)
    slots = cus * (3 if kind == "fp8" else 2)
    B, H, Sq, Sk = 1, 1, 128 * (3 * slots + max(1, slots // 16)), 64 * 120
    g = torch.Generator().manual_seed(cus)
    q = torch.randn(B, H, Sq, 128, generator=g)
    k, v = (torch.randn(B, H, Sk, 128, generator=g) for _ in range(2))
    if kind == "fp8":
        (q8, qd), (k8, kd), (v8, vd) = (O.per_head_quant_ref(t) for t in (q, k, v))
        args = tuple(t.to(gpu) for t in (q8, k8, v8))
        kw = dict(q_descale=qd.to(gpu), k_descale=kd.to(gpu), v_descale=vd.to(gpu))
        qr, kr, vr = O.dequant(q8, qd), O.dequant(k8, kd), O.dequant(v8, vd)
        tol_o, tol_l = 6e-2, 1e-3
    else:
        args, kw = tuple(t.bfloat16().to(gpu) for t in (q, k, v)), {}
        qr, kr, vr = (t.bfloat16() for t in (q, k, v))
        tol_o, tol_l = TOL[torch.bfloat16]
    plan = ops.launch_plan(args[0], args[1])
    assert plan["ranges"] > 0 and plan["whole_tiles"] == 3 * slots
    o, l = ops.attn_fwd(*args, **kw)
    o1, l1 = ops.attn_fwd(*args, balance=False, **kw)
    # every row against the plain launch, probe rows of every head against the oracle
    assert (o.float() - o1.float()).abs().max().item() <= 1e-2 and (l - l1).abs().max().item() <= 1e-5
    rows = torch.arange(0, Sq, 997)
    ro, rl = O.attn_fwd_ref(qr[:, :, rows], kr, vr)
    assert _err(o[:, :, rows.to(gpu)], ro) <= tol_o and _err(l[:, :, rows.to(gpu)], rl) <= tol_l


@pytest.mark.parametrize("kind", ["streamed-or-ranges", "claimed-ranges"])
def test_workspace_counters_between_calls(gpu, sharing_mode, force_rows, kind):
    """The counters at the start of a workspace: a first call on memory full of ones clears them
    itself (workspace_preserved = 0), later calls on the same buffer rely on the fold kernel having
    put them back to zero (workspace_preserved = 1), also when the shape changes in between."""
    if kind == "claimed-ranges":
        force_rows(384)
        q, k, v = _claimed_ranges_problem(gpu, 11)
    else:
        g = torch.Generator(device=gpu).manual_seed(3)
        q, k, v = (torch.randn(1, 3, 4608, 128, generator=g, device=gpu).bfloat16() for _ in range(3))
    plan = ops.launch_plan(q, k)
    assert plan["ranges"] > 0 and plan["counter"] == (1 if kind == "claimed-ranges" or sharing_mode == "streamed" else 0)
    ref_o, ref_l = ops.attn_fwd(q, k, v, balance=False)
    key = (q.device, ops._stream(q.device))
    poisoned = torch.full((plan["workspace_bytes"] + (32 << 20),), 0xFF, dtype=torch.uint8, device=gpu)   # room for the other shape too
    ops._WORKSPACE[key] = [poisoned, 0]
    small = tuple(t[:, :2] for t in (q, k, v))   # another shape on the same buffer in between
    for call in range(4):
        o, l = ops.attn_fwd(q, k, v)
        assert ops._WORKSPACE[key][0] is poisoned and ops._WORKSPACE[key][1] == 1
        assert (o.float() - ref_o.float()).abs().max().item() <= 1e-2 and (l - ref_l).abs().max().item() <= 1e-5, call
        if call == 1:
            so, sl = ops.attn_fwd(*small)
            ro, rl = ops.attn_fwd(*small, balance=False)
            assert (so.float() - ro.float()).abs().max().item() <= 1e-2 and (sl - rl).abs().max().item() <= 1e-5
    torch.cuda.synchronize()
    assert int(poisoned[:16384].max()) == 0   # every counter is back at zero
    del ops._WORKSPACE[key]


def test_workspace_counters_after_a_plain_or_a_failed_first_call(gpu):
    """`workspace_preserved = 1` is legal after ANY successful call that was given the workspace
    with 0: a plain launch clears the counters as well (through the C ABI: balance = 1 with a
    workspace full of ones, then a balanced call that vouches for it).  And the Python wrapper does
    not vouch for a buffer whose first call failed before anything was launched."""
    import ctypes
    g = torch.Generator(device=gpu).manual_seed(9)
    q, k, v = (torch.randn(1, 3, 4608, 128, generator=g, device=gpu).bfloat16() for _ in range(3))
    ref_o, ref_l = ops.attn_fwd(q, k, v, balance=False)
    out, lse = torch.empty_like(q), torch.empty(1, 3, 4608, device=gpu)
    plan = ops._build_attn_plan(q, k, v, 128 ** -0.5, False, None, None, (None, None, None), q.dtype, out, lse, None, False)
    assert plan.need > 0
    a = plan.args
    a.q, a.k, a.v, a.out, a.lse = (t.data_ptr() for t in (q, k, v, out, lse))
    a.stream = ops._stream(gpu)
    ws = torch.full((plan.need,), 0xFF, dtype=torch.uint8, device=gpu)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.workspace_preserved, a.balance = 0, 1          # a plain launch on a fresh workspace
    assert ops._lib.lib().xdit_attn_fwd(ctypes.byref(a)) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, ref_o) and int(ws[:16384].max()) == 0 and int(ws[16384:].min()) == 0xFF
    out.zero_()
    a.workspace_preserved, a.balance = 1, 0          # then a balanced one that vouches for it
    assert ops._lib.lib().xdit_attn_fwd(ctypes.byref(a)) == 0
    torch.cuda.synchronize()
    assert (out.float() - ref_o.float()).abs().max().item() <= 1e-2 and (lse - ref_l).abs().max().item() <= 1e-5
    assert int(ws[:16384].max()) == 0
    # the wrapper: a call that fails validation leaves the buffer unvouched-for
    key = (q.device, ops._stream(q.device))
    poisoned = torch.full((plan.need + 64,), 0xFF, dtype=torch.uint8, device=gpu)
    ops._WORKSPACE[key] = [poisoned, 0]
    bad_q = torch.empty(q.numel() + 1, dtype=q.dtype, device=gpu)[1:].view(q.shape)   # not 16-byte aligned
    with pytest.raises(ValueError, match="aligned"):
        ops.attn_fwd(bad_q, k, v)
    assert ops._WORKSPACE[key][0] is poisoned and ops._WORKSPACE[key][1] == 0
    o, l = ops.attn_fwd(q, k, v)
    assert ops._WORKSPACE[key][1] == 1
    assert (o.float() - ref_o.float()).abs().max().item() <= 1e-2 and (l - ref_l).abs().max().item() <= 1e-5
    del ops._WORKSPACE[key]


@pytest.fixture
def force_rows(monkeypatch):
    """Pins the query rows per workgroup (128 / 256 / 384: 4 / 8 / 12 wavefronts) that the library
    would otherwise pick from the problem size (the rows_per_workgroup field of xdit_attn_args)."""
    def set_rows(rows):
        monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", int(rows))
    return set_rows


@pytest.mark.gpu
@pytest.mark.parametrize("kind,rows,Sk", [("bf16", 384, 256 * 64), ("bf16", 256, 512 * 64), ("bf16", 128, 512 * 64),
                                          ("fp8", 384, 256 * 64)])
def test_claimed_ranges_vs_plain_launch_and_fp32(gpu, force_rows, kind, rows, Sk):
    """Query tiles that leave a long share of KV iterations per workgroup in the last round (at 384
    rows: 384 tiles, 128 of them shared, 128 iterations per workgroup): the bf16 kernel cuts the
    shares into ranges of 64 iterations which the workgroups claim from a counter, at every
    workgroup shape (the fp8 kernel gives every workgroup one range).  The result must match the
    plain launch, a fp32 computation of two heads, and itself on a second call (which workgroup
    takes which range changes nothing).  A secondary check: at this size the reference values
    come from torch on the GPU in fp32, not from the float64 oracle (the oracle-pinned cases of
    the same code path are test_balanced_launch_vs_oracle and test_random_problems_vs_oracle)."""
    force_rows(rows)
    B, H, Sq = 1, 12, 32 * 384
    g = torch.Generator(device=gpu).manual_seed(77)
    q, k, v = (torch.randn(B, H, n, 128, generator=g, device=gpu) for n in (Sq, Sk, Sk))
    if kind == "fp8":
        (q8, qd), (k8, kd), (v8, vd) = (ops.fp8_quant(t.to(torch.bfloat16)) for t in (q, k, v))
        args, kw = (q8, k8, v8), dict(q_descale=qd, k_descale=kd, v_descale=vd)
        deq = lambda t, d: t.float() * d[:, :, None, None]
        qf, kf, vf = deq(q8, qd), deq(k8, kd), deq(v8, vd)
        tol_o, tol_l = 6e-2, 1e-3
    else:
        args, kw = tuple(t.to(torch.bfloat16) for t in (q, k, v)), {}
        qf, kf, vf = (t.float() for t in args)
        tol_o, tol_l = TOL[torch.bfloat16]
    plan = ops.launch_plan(args[0], args[1])
    assert plan["rows_per_workgroup"] == rows and plan["ranges"] > 0 and plan["counter"] == (kind == "bf16")
    o, l = ops.attn_fwd(*args, **kw)
    o1, l1 = ops.attn_fwd(*args, balance=False, **kw)
    assert (o.float() - o1.float()).abs().max().item() <= 1e-2 and (l - l1).abs().max().item() <= 1e-5
    for h in (0, H - 1):
        s = (qf[:, h] @ kf[:, h].transpose(-1, -2)) * 128 ** -0.5
        ro, rl = torch.softmax(s, -1) @ vf[:, h], torch.logsumexp(s, -1)
        assert (o[:, h].float() - ro).abs().max().item() <= tol_o
        assert (l[:, h] - rl).abs().max().item() <= tol_l
    o2, l2 = ops.attn_fwd(*args, **kw)
    assert torch.equal(o, o2) and torch.equal(l, l2)


@pytest.mark.parametrize("rows", [128, 256, 384])
@pytest.mark.parametrize("kind", ["bf16", "fp16", "fp8", "bf16-d64", "fp16-d64", "bf16-d72", "fp16-d40", "fp16-d96", "bf16-d120", "bf16-d8"])
@pytest.mark.parametrize("B,H,Sq,Sk,Sk2", [
    (1, 2, 1000, 777, 0),       # several workgroups per head, partial last query tile and KV tile
    (1, 1, 385, 8192, 0),       # balanced launch: KV ranges shared between workgroups
    (1, 3, 700, 5000, 90),      # balanced launch with a second KV segment
    (2, 2, 50, 64, 1),          # fewer query rows than one workgroup covers
])
def test_workgroup_shapes_vs_oracle(gpu, force_rows, rows, kind, B, H, Sq, Sk, Sk2):
    """Every workgroup shape of the 16-bit (built for head_dim 128 and 64, also on tensors of a
    smaller head_dim) and fp8 kernels, with and without the balanced launch, against the oracle on
    the same inputs."""
    force_rows(rows)
    D = int(kind.split("-d")[1]) if "-d" in kind else 128
    kind = kind.split("-")[0]
    g = torch.Generator().manual_seed(rows + Sq + Sk)
    mk = lambda n: torch.randn(B, H, n, D, generator=g)
    q, k, v = mk(Sq), mk(Sk), mk(Sk)
    k2, v2 = (mk(Sk2), mk(Sk2)) if Sk2 else (None, None)
    dev = lambda t: None if t is None else t.to(gpu)
    if kind == "fp8":
        kall = k if k2 is None else torch.cat([k, k2], 2)
        vall = v if v2 is None else torch.cat([v, v2], 2)
        (q8, qd), (k8, kd), (v8, vd) = (O.per_head_quant_ref(t) for t in (q, kall, vall))
        ro, rl = O.attn_fwd_ref(O.dequant(q8, qd), O.dequant(k8, kd), O.dequant(v8, vd))
        kw = dict(q_descale=dev(qd), k_descale=dev(kd), v_descale=dev(vd))
        if Sk2:
            kw.update(k2=dev(k8[:, :, Sk:].contiguous()), v2=dev(v8[:, :, Sk:].contiguous()))
            k8, v8 = k8[:, :, :Sk].contiguous(), v8[:, :, :Sk].contiguous()
        args = (dev(q8), dev(k8), dev(v8))
        tol_o, tol_l = 6e-2, 1e-3
    else:
        dt = torch.bfloat16 if kind == "bf16" else torch.float16
        q, k, v = q.to(dt), k.to(dt), v.to(dt)
        kall, vall = k, v
        kw = {}
        if Sk2:
            k2, v2 = k2.to(dt), v2.to(dt)
            kall, vall = torch.cat([k, k2], 2), torch.cat([v, v2], 2)
            kw.update(k2=dev(k2), v2=dev(v2))
        ro, rl = O.attn_fwd_ref(q, kall, vall)
        args = (dev(q), dev(k), dev(v))
        tol_o, tol_l = TOL[dt]
    assert ops.launch_plan(args[0], args[1], k2=kw.get("k2"))["rows_per_workgroup"] == rows
    o, l = ops.attn_fwd(*args, **kw)
    o1, l1 = ops.attn_fwd(*args, balance=False, **kw)
    assert _err(o, ro) <= tol_o and _err(l, rl) <= tol_l
    assert _err(o1, ro) <= tol_o and _err(l1, rl) <= tol_l


# ---------------------------------------------------------------------------- named configurations
def test_c1_pixart512_fp32_full(gpu):
    z = np.load(os.path.join(GOLD, "c1_pixart512.npz"))
    c = O.make_config("c1_pixart512")
    o, l = ops.attn_fwd(c["q"].to(gpu), c["k"].to(gpu), c["v"].to(gpu), softmax_scale=72 ** -0.5)
    assert _err(o[:, :, ::37], torch.from_numpy(z["out_rows"])) <= 2e-5
    assert _err(l, torch.from_numpy(z["lse"])) <= 2e-5
    # and against the op the reference's SDPA_MATH backend calls, on the CPU
    mo, _ = torch.ops.aten._scaled_dot_product_attention_math(c["q"], c["k"], c["v"])
    assert _err(o, mo) <= 2e-5


@pytest.fixture(scope="module")
def flux(gpu):
    c = O.make_config("c2_flux1024")
    z = np.load(os.path.join(GOLD, "c2_flux1024_rows.npz"))
    d = {n: c[n].to(gpu) for n in "qkv"}
    d["rows"] = torch.from_numpy(z["rows"]).to(gpu)
    d["ref_out"], d["ref_lse"] = torch.from_numpy(z["out"]), torch.from_numpy(z["lse"])
    return d


def test_c2_flux1024_single_pass(gpu, sharing_mode, flux):
    plan = ops.launch_plan(flux["q"], flux["k"])
    assert plan["streamed"] == (sharing_mode == "streamed") and plan["ranges"] == 256
    o, l = ops.attn_fwd(flux["q"], flux["k"], flux["v"])
    assert _err(o[:, :, flux["rows"]], flux["ref_out"]) <= 2e-2
    assert _err(l[:, :, flux["rows"]], flux["ref_lse"]) <= 1e-3
    lse_tol = 0 if sharing_mode == "deterministic" else 1e-5
    # determinism and layout invariance: bit-identical results (to rounding under streamed sharing)
    o2, l2 = ops.attn_fwd(flux["q"], flux["k"], flux["v"])
    assert _same(o, o2, sharing_mode) and (l - l2).abs().max().item() <= lse_tol
    tb = lambda t: t.transpose(1, 2).contiguous().transpose(1, 2)
    o3, l3 = ops.attn_fwd(tb(flux["q"]), tb(flux["k"]), tb(flux["v"]))
    assert _same(o, o3, sharing_mode) and (l - l3).abs().max().item() <= lse_tol
    # the registry adapter and USP return the same thing
    o4, l4 = AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355](flux["q"], flux["k"], flux["v"], 0.0, False)
    assert _same(o, o4, sharing_mode) and (l - l4).abs().max().item() <= lse_tol
    assert _same(o, usp.USP(flux["q"], flux["k"], flux["v"]), sharing_mode)
    # whole query tiles do not depend on the sharing: the first 256 tiles of 384 rows are bit-identical
    od, _ = ops.attn_fwd(flux["q"], flux["k"], flux["v"], streamed=False)
    flat = lambda t: t.reshape(-1, 128)[: 256 * 384]
    assert torch.equal(flat(o), flat(od))


@pytest.mark.parametrize("order", [None, [0, 1, 2, 3]])
def test_c3_flux_ring_of_4_equals_single_pass(gpu, flux, order):
    o, l = ops.attn_fwd(flux["q"], flux["k"], flux["v"])
    fn = usp._get_attention_function()
    merged = usp.ring_attn(fn, flux["q"], flux["k"], flux["v"], ring_chunks=4, order=order)
    assert merged.dtype == torch.bfloat16
    assert _err(merged[:, :, flux["rows"]], flux["ref_out"]) <= 2e-2
    assert _err(merged, o.cpu()) <= 2e-2
    # legacy BSHD loop with update_out_and_lse, returning the lse as well
    qb, kb, vb = (flux[n].transpose(1, 2).contiguous() for n in "qkv")
    ob, lb, _ = ring.xdit_ring_flash_attn_func(qb, kb, vb, return_attn_probs=True, group=ring.LocalRing(4))
    assert ob.shape == qb.shape and lb.shape == (1, 24, 4608)
    assert _err(ob.transpose(1, 2)[:, :, flux["rows"]], flux["ref_out"]) <= 2e-2
    assert _err(lb[:, :, flux["rows"]], flux["ref_lse"]) <= 1e-3
    assert _err(lb, l.cpu()) <= 1e-3


def test_c4_hunyuan720p_shard_full_size(gpu):
    """(1, 3, 119056, 128) bf16: probe rows against the oracle over the full K/V, plus
    chunk-fold and key-permutation invariance at full size."""
    c = O.make_config("c4_hunyuan720p_shard")
    S = c["q"].shape[2]
    assert S == 119056
    rows = [0, 1, 127, 128, 4097, 60000, 118799, 118800, 119040, 119055]
    ro, rl = O.attn_rows_ref(c["q"], c["k"], c["v"], rows)
    q, k, v = (c[n].to(gpu) for n in "qkv")
    o, l = ops.attn_fwd(q, k, v)
    assert _err(o[:, :, rows], ro) <= 2e-2 and _err(l[:, :, rows], rl) <= 1e-3
    assert torch.isfinite(o.float()).all() and torch.isfinite(l).all()
    # fold of two unequal KV chunks (video | text, as a joint ring step would see them)
    o1, l1 = ops.attn_fwd(q, k[:, :, :118800], v[:, :, :118800])
    o2, l2 = ops.attn_fwd(q, k[:, :, 118800:], v[:, :, 118800:])
    m = usp.SDPAMerger()
    m.step(o1, l1)
    m.step(o2, l2, final_step=True)
    mo, ml = m.results()
    assert _err(mo, o.cpu()) <= 2e-2 and _err(ml, l.cpu()) <= 1e-3
    # two-segment call == single call, and key order does not matter
    o3, l3 = ops.attn_fwd(q, k[:, :, 118800:], v[:, :, 118800:], k2=k[:, :, :118800], v2=v[:, :, :118800])
    assert _err(o3, o.cpu()) <= 2e-2 and _err(l3, l.cpu()) <= 1e-3


def test_c5_wan720p_shard_fp8_full_size(gpu):
    """(1, 5, 75600, 128) fp8 e4m3fn + per-head scales -> bf16 out, fp32 lse."""
    c = O.make_config("c5_wan720p_shard_fp8")
    assert c["q"].shape == (1, 5, 75600, 128)
    rows = [0, 31, 32, 1000, 40000, 75519, 75520, 75599]
    dq, dk, dv = (O.dequant(c[n], c[n + "_descale"]) for n in "qkv")
    ro, rl = O.attn_rows_ref(dq, dk, dv, rows)
    args = {n: c[n].to(gpu) for n in c}
    o, l = ops.attn_fwd(args["q"], args["k"], args["v"], q_descale=args["q_descale"],
                        k_descale=args["k_descale"], v_descale=args["v_descale"])
    assert o.dtype == torch.bfloat16 and l.dtype == torch.float32
    assert _err(o[:, :, rows], ro) <= 6e-2 and _err(l[:, :, rows], rl) <= 1e-3
    assert torch.isfinite(o.float()).all() and torch.isfinite(l).all()


@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_fp8_golden_s2048(gpu, layout):
    z = np.load(os.path.join(GOLD, "c5_fp8_s2048_rows.npz"))
    c = O.make_config("c5_wan720p_shard_fp8", S=2048)
    rows = torch.from_numpy(z["rows"])
    lay = lambda t: t.view(torch.uint8).transpose(1, 2).contiguous().transpose(1, 2).view(torch.float8_e4m3fn) if layout == "bshd" else t
    o, l = ops.attn_fwd(lay(c["q"]).to(gpu), lay(c["k"]).to(gpu), lay(c["v"]).to(gpu),
                        q_descale=c["q_descale"].to(gpu), k_descale=c["k_descale"].to(gpu), v_descale=c["v_descale"].to(gpu),
                        out_dtype=torch.float16)
    assert o.dtype == torch.float16
    assert _err(o[:, :, rows], torch.from_numpy(z["out"])) <= 6e-2
    assert _err(l[:, :, rows], torch.from_numpy(z["lse"])) <= 1e-3


@pytest.mark.parametrize("Sq,Sk", [(1, 1), (100, 63), (129, 130), (64, 1000)])
def test_fp8_small_vs_oracle(gpu, Sq, Sk):
    """A secondary check on inputs three times wider than the benchmark's: outputs reach several
    units, so the 6e-2 bar is applied relative to the largest output value where that exceeds 1.
    The absolute 6e-2 bar is asserted by test_fp8_golden_s2048 and the full-size Wan shard."""
    g = torch.Generator().manual_seed(Sq + Sk)
    q, k, v = (torch.randn(2, 2, n, 128, generator=g) * 3 for n in (Sq, Sk, Sk))
    (q8, qd), (k8, kd), (v8, vd) = (O.per_head_quant_ref(t) for t in (q, k, v))
    ro, rl = O.attn_fwd_ref(O.dequant(q8, qd), O.dequant(k8, kd), O.dequant(v8, vd))
    o, l = ops.attn_fwd(q8.to(gpu), k8.to(gpu), v8.to(gpu), q_descale=qd.to(gpu), k_descale=kd.to(gpu), v_descale=vd.to(gpu))
    # logits here have a standard deviation of about 9: few keys carry the mass, which is the
    # hard case for an fp8 P matrix
    assert _err(o, ro) <= 6e-2 * max(1.0, ro.abs().max().item()) and _err(l, rl) <= 1e-3


@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
@pytest.mark.parametrize("rows", [128, 256, 384])
@pytest.mark.parametrize("Sq,Sk,Sk2", [(1, 1, 0), (100, 63, 0), (129, 130, 50), (300, 1000, 1), (64, 64, 64)])
def test_fp8_head_dim_64_vs_oracle(gpu, force_rows, layout, rows, Sq, Sk, Sk2):
    """The fp8 forward at head_dim 64 (SD3, CogVideoX, the audio stream of LTX2: what the
    reference's hybrid bf16/fp8 schedule hands its fp8 backend for those models): one contraction
    step of 64 for S^T, two 32-row blocks of O^T.  Every workgroup shape, both memory layouts,
    ragged sizes and a second KV segment, against the oracle on the dequantised inputs at the
    absolute 6e-2 / 1e-3 bars."""
    force_rows(rows)
    g = torch.Generator().manual_seed(Sq + 7 * Sk + Sk2)
    q, k, v = (torch.randn(2, 3, n, 64, generator=g) for n in (Sq, Sk + Sk2, Sk + Sk2))
    (q8, qd), (k8, kd), (v8, vd) = (O.per_head_quant_ref(t) for t in (q, k, v))
    ro, rl = O.attn_fwd_ref(O.dequant(q8, qd), O.dequant(k8, kd), O.dequant(v8, vd))
    dev = lambda t: _layout(t.view(torch.uint8), layout, gpu).view(torch.float8_e4m3fn)
    kw = dict(q_descale=qd.to(gpu), k_descale=kd.to(gpu), v_descale=vd.to(gpu))
    if Sk2:
        kw.update(k2=dev(k8[:, :, Sk:].contiguous()), v2=dev(v8[:, :, Sk:].contiguous()))
    o, l = ops.attn_fwd(dev(q8), dev(k8[:, :, :Sk].contiguous()), dev(v8[:, :, :Sk].contiguous()), **kw)
    assert o.dtype == torch.bfloat16 and _err(o, ro) <= 6e-2 and _err(l, rl) <= 1e-3


def test_fp8_head_dim_64_sd3_shape_balanced_and_ring_step(gpu, monkeypatch):
    """SD3-1024 joint attention (B=2, H=24, S=4250, head_dim 64) in fp8: the library's launch
    (balanced) against the plain launch on every row and against the oracle on probe rows; and
    the fused ring step at head_dim 64 against forward + merge, bit for bit."""
    g = torch.Generator(device=gpu).manual_seed(64)
    q, k, v = (torch.randn(2, 24, 4250, 64, generator=g, device=gpu) for _ in range(3))
    (q8, qd), (k8, kd), (v8, vd) = (ops.fp8_quant(t) for t in (q, k, v))
    kw = dict(q_descale=qd, k_descale=kd, v_descale=vd)
    assert ops.launch_plan(q8, k8)["ranges"] > 0
    o, l = ops.attn_fwd(q8, k8, v8, **kw)
    po, pl = ops.attn_fwd(q8, k8, v8, balance=False, **kw)
    assert (o.float() - po.float()).abs().max().item() <= 1e-2 and (l - pl).abs().max().item() <= 1e-5
    probe = torch.arange(0, 4250, 331)
    ro, rl = O.attn_fwd_ref(O.dequant(q8.cpu(), qd.cpu())[:, :, probe], O.dequant(k8.cpu(), kd.cpu()), O.dequant(v8.cpu(), vd.cpu()))
    assert _err(o[:, :, probe.to(gpu)], ro) <= 6e-2 and _err(l[:, :, probe.to(gpu)], rl) <= 1e-3
    monkeypatch.setitem(ops.TUNING, "streamed", 0)
    acc_o, acc_l = torch.full((2, 24, 4250, 64), float("nan"), device=gpu), torch.full((2, 24, 4250), float("nan"), device=gpu)
    ref_o, ref_l = torch.empty_like(acc_o), torch.empty_like(acc_l)
    fin, ref_fin = torch.empty(2, 24, 4250, 64, dtype=torch.bfloat16, device=gpu), torch.empty(2, 24, 4250, 64, dtype=torch.bfloat16, device=gpu)
    for i, (a, b) in enumerate(((0, 2000), (2000, 4250))):
        ks, vs = k8[:, :, a:b], v8[:, :, a:b]
        ops.attn_fwd_accumulate(q8, ks, vs, acc_o, acc_l, first=i == 0, final_out=fin if i else None, **kw)
        bo, bl = ops.attn_fwd(q8, ks, vs, **kw)
        ops.lse_merge(ref_o, ref_l, bo, bl, first=i == 0, final_out=ref_fin if i else None)
        assert torch.equal(acc_o, ref_o) and torch.equal(acc_l, ref_l), i
    assert torch.equal(fin, ref_fin)
    assert (fin.float() - o.float()).abs().max().item() <= 2e-2 and (acc_l - l).abs().max().item() <= 1e-4   # two chunks = single pass


@pytest.mark.parametrize("balance", [1, 2])
@pytest.mark.parametrize("rows", [128, 256, 384])
@pytest.mark.parametrize("kind,D", [("bf16", 128), ("bf16", 64), ("fp16", 96), ("fp8", 128)])
def test_every_launch_option_vs_oracle(gpu, monkeypatch, kind, D, rows, balance):
    """The six ways a problem can be launched -- 128, 256 or 384 query rows per workgroup, as a plain
    launch or with the last round balanced -- each forced through the tuning fields of
    xdit_attn_args on a problem where all six exist (5 heads of 1000 rows on 1100 + 100 keys: no
    workgroup shape fills the chip, so every query tile is shared), against the float64 oracle.
    The default (whichever of the six the library's time estimate picks) is checked too."""
    g = torch.Generator().manual_seed(D + rows + balance)
    q, k, v, k2, v2 = (torch.randn(1, 5, n, D, generator=g) for n in (1000, 1100, 1100, 100, 100))
    if kind == "fp8":
        (q, qd), (kk, kd), (vv, vd) = (O.per_head_quant_ref(t) for t in (q, torch.cat([k, k2], 2), torch.cat([v, v2], 2)))
        k, k2, v, v2 = kk[:, :, :1100], kk[:, :, 1100:], vv[:, :, :1100], vv[:, :, 1100:]
        ro, rl = O.attn_fwd_ref(O.dequant(q, qd), O.dequant(kk, kd), O.dequant(vv, vd))
        kw = dict(q_descale=qd.to(gpu), k_descale=kd.to(gpu), v_descale=vd.to(gpu))
        tol = (6e-2, 1e-3)
    else:
        dtype = torch.bfloat16 if kind == "bf16" else torch.float16
        q, k, v, k2, v2 = (t.to(dtype) for t in (q, k, v, k2, v2))
        ro, rl = O.attn_fwd_ref(q, torch.cat([k, k2], 2), torch.cat([v, v2], 2))
        kw, tol = {}, TOL[dtype]
    dq, dk, dv, dk2, dv2 = (t.to(gpu) for t in (q, k, v, k2, v2))
    for forced in (True, False):
        monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", rows if forced else 0)
        monkeypatch.setitem(ops.TUNING, "balance", balance if forced else 0)
        plan = ops.launch_plan(dq, dk, k2=dk2)
        if forced:
            assert plan["rows_per_workgroup"] == rows and (plan["ranges"] > 0) == (balance == 2), plan
        o, l = ops.attn_fwd(dq, dk, dv, k2=dk2, v2=dv2, **kw)
        assert _err(o, ro) <= tol[0] and _err(l, rl) <= tol[1], (forced, plan)


# ---------------------------------------------------------------------------- merge
@pytest.mark.parametrize("block_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_merge_vs_oracle(gpu, block_dtype, layout):
    B, H, S, D = 2, 3, 257, 128
    g = torch.Generator().manual_seed(21)
    out = torch.randn(B, H, S, D, generator=g)
    lse = torch.randn(B, H, S, generator=g) * 3
    bo = torch.randn(B, H, S, D, generator=g).to(block_dtype)
    bl = torch.randn(B, H, S, generator=g) * 3
    ro, rl = O.merge_ref(out, lse, bo, bl)
    ao = _layout(out, layout, gpu)
    al = lse.to(gpu) if layout == "bhsd" else lse.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    fo = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=gpu)
    ops.lse_merge(ao, al, _layout(bo, layout, gpu), bl.to(gpu), final_out=fo)
    assert _err(ao, ro) <= 2e-6 and _err(al, rl) <= 2e-6
    assert torch.equal(fo, ao.bfloat16())


@pytest.mark.parametrize("D", [72, 40, 104, 512])
def test_merge_rows_that_do_not_fill_a_wavefront(gpu, D):
    """head_dim / 8 that does not divide 64 (72 is PixArt's, the head_dim of the fp32 ring): with a
    flat thread -> chunk map a row straddles two wavefronts or workgroups and its later lanes can
    read the log-sum-exp the first lane has already replaced.  2^17 rows fill the chip several
    times over, so late workgroups exist; folds are checked against the oracle row by row, twice
    over on the same accumulator."""
    B, H, S = 1, 4, 1 << 15
    g = torch.Generator().manual_seed(D)
    acc_o, blk1, blk2 = (torch.randn(B, H, S, D, generator=g) for _ in range(3))
    acc_l, l1, l2 = (torch.randn(B, H, S, generator=g) * 3 for _ in range(3))
    mo, ml = O.merge_ref(acc_o, acc_l, blk1, l1)
    mo2, ml2 = O.merge_ref(mo, ml, blk2.bfloat16(), l2)
    a_o, a_l = acc_o.to(gpu), acc_l.to(gpu)
    ops.lse_merge(a_o, a_l, blk1.to(gpu), l1.to(gpu))
    assert _err(a_o, mo) <= 2e-5 and _err(a_l, ml) <= 2e-5
    fin = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=gpu)
    ops.lse_merge(a_o, a_l, blk2.bfloat16().to(gpu), l2.to(gpu), final_out=fin)
    assert _err(a_o, mo2) <= 4e-5 and _err(a_l, ml2) <= 4e-5
    assert _err(fin, mo2) <= 2.0 ** -8 * max(1.0, mo2.abs().max().item())


def test_merge_first_call_and_special_values(gpu):
    B, H, S, D = 1, 2, 64, 64
    bo = torch.randn(B, H, S, D).bfloat16().to(gpu)
    bl = torch.randn(B, H, S).to(gpu)
    ao = torch.full((B, H, S, D), float("nan"), device=gpu)
    al = torch.full((B, H, S), float("nan"), device=gpu)
    ops.lse_merge(ao, al, bo, bl, first=True)
    assert torch.equal(ao, bo.float()) and torch.equal(al, bl)
    # a block with lse = -inf leaves the accumulator unchanged
    before_o, before_l = ao.clone(), al.clone()
    ops.lse_merge(ao, al, torch.randn_like(bo), torch.full_like(bl, float("-inf")))
    assert torch.equal(ao, before_o) and torch.equal(al, before_l)
    # equal lse: mean and lse + ln 2
    bo2 = torch.randn(B, H, S, D, device=gpu)
    ops.lse_merge(ao, al, bo2, before_l.clone())
    assert _err(ao, 0.5 * (before_o + bo2).cpu()) <= 1e-6 and _err(al, (before_l + np.log(2.0)).cpu()) <= 1e-6


def test_merge_golden_fold(gpu):
    z = np.load(os.path.join(GOLD, "merge_fold.npz"))
    ao = torch.from_numpy(z["out"]).float().to(gpu)
    al = torch.from_numpy(z["lse"]).float().to(gpu)
    ops.lse_merge(ao, al, torch.from_numpy(z["block_out"]).float().to(gpu), torch.from_numpy(z["block_lse"]).float().to(gpu))
    assert _err(ao, torch.from_numpy(z["new_out"])) <= 2e-6 and _err(al, torch.from_numpy(z["new_lse"])) <= 2e-6


def test_update_out_and_lse_matches_oracle_layout(gpu):
    B, S, H, D = 2, 100, 3, 128
    g = torch.Generator().manual_seed(5)
    blocks = [(torch.randn(B, S, H, D, generator=g).bfloat16(), torch.randn(B, H, S, generator=g) * 2) for _ in range(3)]
    out = lse = rout = rlse = None
    for bo, bl in blocks:
        out, lse = ring.update_out_and_lse(out, lse, bo.to(gpu), bl.to(gpu))
        rout, rlse = O.update_out_and_lse_ref(rout, rlse, bo, bl, dtype=torch.float64)
    assert out.shape == (B, S, H, D) and lse.shape == (B, S, H, 1) and out.dtype == torch.float32
    assert _err(out, rout) <= 5e-6 and _err(lse, rlse) <= 5e-6

@pytest.mark.gpu
@pytest.mark.parametrize("rows", [128, 256, 384])
@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 72), (torch.float16, 88), (torch.bfloat16, 40), (torch.float16, 16)])
def test_smaller_head_dim_touches_only_its_columns(gpu, force_rows, rows, dtype, D):
    """Tensors of a head_dim below the one the 16-bit kernel is built for: the kernel must neither
    read nor write the columns they do not have.  q, k, v and out are views of wider tensors whose
    other columns hold NaN (a read would poison the result, a write would clear the NaN)."""
    force_rows(rows)
    W = 136
    B, H, Sq = 1, 2, 500
    g = torch.Generator().manual_seed(rows + D)
    for Sk, balance in ((333, True), (8192, True), (8192, False)):
        wide = lambda n: torch.full((B, H, n, W), float("nan"), dtype=dtype, device=gpu)
        qw, kw_, vw, ow = wide(Sq), wide(Sk), wide(Sk), wide(Sq)
        q, k, v = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk))
        qw[..., 8:8 + D], kw_[..., 16:16 + D], vw[..., :D] = q.to(gpu), k.to(gpu), v.to(gpu)
        out = ow[..., 24:24 + D]
        o, l = ops.attn_fwd(qw[..., 8:8 + D], kw_[..., 16:16 + D], vw[..., :D], out=out, balance=balance)
        ro, rl = O.attn_fwd_ref(q, k, v)
        assert _err(out, ro) <= TOL[dtype][0] and _err(l, rl) <= TOL[dtype][1]
        assert torch.isnan(ow[..., :24]).all() and torch.isnan(ow[..., 24 + D:]).all()
        # the same through the fused ring step: accumulator and final output inside NaN frames
        aw = torch.full((B, H, Sq, W), float("nan"), device=gpu)
        acc_o, acc_l = aw[..., 4:4 + D], torch.empty(B, H, Sq, device=gpu)
        fw = wide(Sq)
        ops.attn_fwd_accumulate(qw[..., 8:8 + D], kw_[..., 16:16 + D], vw[..., :D], acc_o, acc_l, first=True, final_out=fw[..., 8:8 + D])
        po, pl = (out, l) if not balance else ops.attn_fwd(qw[..., 8:8 + D], kw_[..., 16:16 + D], vw[..., :D], balance=False)
        assert torch.equal(fw[..., 8:8 + D], po) and torch.equal(acc_l, pl) and torch.equal(acc_o, po.float())
        assert torch.isnan(aw[..., :4]).all() and torch.isnan(aw[..., 4 + D:]).all()
        assert torch.isnan(fw[..., :8]).all() and torch.isnan(fw[..., 8 + D:]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [128, 256, 384])
@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 72), (torch.float16, 88)])
def test_smaller_head_dim_in_a_balanced_launch(gpu, monkeypatch, rows, dtype, D):
    """A head_dim below the kernel's own (72, 88 on the kernel built for 128) in a balanced launch,
    where a workgroup runs several segments one after the other: between two segments the LDS
    columns that no tile load writes are cleared again, which must wait until every wavefront is
    done with its output staging block in the same memory (a workgroup that did not wait stored
    zeros, or the neighbour's values, in some rows: a regression test).  Every row of three calls
    against the plain launch (one workgroup per query tile) and probe rows against the oracle."""
    monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", rows)
    monkeypatch.setitem(ops.TUNING, "balance", 2)
    g = torch.Generator(device=gpu).manual_seed(D)
    q, k, v = (torch.randn(1, 24, 4608, D, generator=g, device=gpu).to(dtype) for _ in range(3))
    assert ops.launch_plan(q, k)["ranges"] > 0
    plain_o, plain_l = ops.attn_fwd(q, k, v, balance=False)
    for call in range(3):
        out = torch.full_like(q, float("nan"))
        lse = torch.full((1, 24, 4608), float("nan"), device=gpu)
        ops.attn_fwd(q, k, v, out=out, lse=lse)
        assert (out.float() - plain_o.float()).abs().max().item() <= 1e-2 and (lse - plain_l).abs().max().item() <= 1e-5, call
    probe = torch.arange(0, 4608, 211)
    ro, rl = O.attn_fwd_ref(q.cpu()[:, :, probe], k.cpu(), v.cpu())
    assert _err(out[:, :, probe.to(gpu)], ro) <= 2e-2 and _err(lse[:, :, probe.to(gpu)], rl) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(8))
def test_random_problems_vs_oracle(gpu, monkeypatch, seed):
    """Random small problems over everything a call can vary: dtype, head_dim (every multiple of 8
    up to 128), ragged lengths, a second KV segment, memory layout per tensor, softmax scale,
    workgroup shape (forced or chosen by the library), balanced or plain launch, and the fused
    ring step on top of an earlier block.  Every result is checked against the oracle."""
    import random
    rnd = random.Random(1000 + seed)
    g = torch.Generator().manual_seed(seed)
    for case in range(8):
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        D = 8 * rnd.randint(1, 16)
        B, H = rnd.randint(1, 2), rnd.randint(1, 4)
        Sq = rnd.choice([1, 7, 33, 128, 129, 300, 385, 700])
        Sk = rnd.choice([1, 5, 64, 65, 200, 1000, 3000])
        Sk2 = rnd.choice([0, 0, 1, 77, 256])
        rows = rnd.choice([None, 128, 256, 384])
        balance = rnd.random() < 0.7
        scale = rnd.choice([None, 0.05, 0.2])
        if rows is None:
            monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", 0)
        else:
            monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", int(rows))
        mk = lambda n: torch.randn(B, H, n, D, generator=g).to(dtype)
        q, k, v = mk(Sq), mk(Sk), mk(Sk)
        k2, v2 = (mk(Sk2), mk(Sk2)) if Sk2 else (None, None)
        lay = lambda t: None if t is None else _layout(t, rnd.choice(["bhsd", "bshd"]), gpu)
        what = (seed, case, dtype, D, B, H, Sq, Sk, Sk2, rows, balance, scale)
        kall, vall = (k, v) if not Sk2 else (torch.cat([k, k2], 2), torch.cat([v, v2], 2))
        ro, rl = O.attn_fwd_ref(q, kall, vall, scale)
        qd, kd, vd, k2d, v2d = lay(q), lay(k), lay(v), lay(k2), lay(v2)
        o, l = ops.attn_fwd(qd, kd, vd, softmax_scale=scale, k2=k2d, v2=v2d, balance=balance)
        assert _err(o, ro) <= TOL[dtype][0] and _err(l, rl) <= TOL[dtype][1], what
        if ops.fused_ring_step_supported(qd):
            # an earlier block (the first Sk keys alone), then this call folded on top of it
            bo, bl = ops.attn_fwd(qd, kd, vd, softmax_scale=scale)
            acc_o, acc_l = torch.empty(B, H, Sq, D, device=gpu), torch.empty(B, H, Sq, device=gpu)
            ops.lse_merge(acc_o, acc_l, bo, bl, first=True)
            fin = torch.empty(B, H, Sq, D, dtype=dtype, device=gpu)
            ops.attn_fwd_accumulate(qd, kd, vd, acc_o, acc_l, final_out=fin, softmax_scale=scale, k2=k2d, v2=v2d)
            r1o, r1l = O.attn_fwd_ref(q, k, v, scale)
            mo, ml = O.merge_ref(r1o.to(dtype).double(), r1l, ro.to(dtype), rl)
            # two roundings to the 16-bit type (the block, then the result) on values that are not
            # averages of many keys here and can reach 4-5 (half a unit in the last place of a bf16
            # value in [4, 8) is 0.0156): 2^-7 relative to the largest value, where that is above 2e-2
            tol = max(2e-2, 2.0 ** -7 * mo.abs().max().item())
            assert _err(acc_o, mo) <= tol and _err(acc_l, ml) <= 1e-3 and _err(fin, mo) <= tol, what


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(6))
def test_random_problems_planned_for_few_compute_units(gpu, monkeypatch, seed):
    """Random small problems launched as if the chip had 3 to 24 compute units (the cu_count field
    of xdit_attn_args), so that they run in several rounds, with balanced last rounds, ranges taken
    from the counter, streamed sharing and the fold inside the ring step, in bf16, fp16 and fp8
    (head_dim 64 and 128) with ragged lengths, a second KV segment and both layouts.  Checked: the
    oracle's values; the same bits from a second call and from the entry point that allocates
    nothing (fixed work geometry); the ring step against forward + merge, bit for bit wherever the
    two launches cut the KV iterations the same way."""
    import random
    rnd = random.Random(4000 + seed)
    g = torch.Generator().manual_seed(100 + seed)
    seen = {"balanced": 0, "ring_balanced": 0}
    for case in range(6):
        kind = rnd.choice(["bf16", "fp16", "fp8", "fp8"])
        dtype = torch.float16 if kind == "fp16" else torch.bfloat16
        D = rnd.choice([64, 128]) if kind == "fp8" else 8 * rnd.randint(1, 16)
        B, H = rnd.randint(1, 2), rnd.randint(1, 6)
        Sq = rnd.choice([129, 300, 385, 700, 1153])
        Sk = rnd.choice([65, 1000, 1152, 3000, 9000])
        Sk2 = rnd.choice([0, 1, 77, 256])
        if Sk == 9000:   # long shares (ranges from the counter): keep the oracle's work small
            B, H = 1, min(H, 3)
        tune = {"rows_per_workgroup": rnd.choice([0, 128, 256, 384]), "balance": rnd.choice([0, 2, 2]),
                "cu_count": rnd.choice([3, 4, 8, 16, 24]), "streamed": rnd.choice([0, 0, 1])}
        for name, value in tune.items():
            monkeypatch.setitem(ops.TUNING, name, value)
        what = (seed, case, kind, D, B, H, Sq, Sk, Sk2, tune)
        mk = lambda n: torch.randn(B, H, n, D, generator=g)
        q, k, v = mk(Sq), mk(Sk), mk(Sk)
        k2, v2 = (mk(Sk2), mk(Sk2)) if Sk2 else (None, None)
        lay = lambda t: None if t is None else _layout(t, rnd.choice(["bhsd", "bshd"]), gpu)
        kw = {}
        if kind == "fp8":
            q8, qs = ops.fp8_quant(q.to(gpu))
            if Sk2:
                k8, j8, ks = ops.fp8_quant(k.to(gpu), x2=k2.to(gpu))
                v8, w8, vs = ops.fp8_quant(v.to(gpu), x2=v2.to(gpu))
            else:
                (k8, ks), (v8, vs), j8, w8 = ops.fp8_quant(k.to(gpu)), ops.fp8_quant(v.to(gpu)), None, None
            deq = lambda t, sc: None if t is None else O.dequant(t.cpu(), sc.cpu())
            qr, kr, vr, k2r, v2r = deq(q8, qs), deq(k8, ks), deq(v8, vs), deq(j8, ks), deq(w8, vs)
            ins = [t if t is None else lay(t.cpu().view(torch.uint8)).view(torch.float8_e4m3fn) for t in (q8, k8, v8, j8, w8)]
            kw = dict(q_descale=qs, k_descale=ks, v_descale=vs, out_dtype=dtype)
            tol_rel, tol_abs = 2.0 ** -4, 6e-2   # one unit in the last place of an e4m3 probability
        else:
            qr, kr, vr = q.to(dtype), k.to(dtype), v.to(dtype)
            k2r, v2r = (k2.to(dtype), v2.to(dtype)) if Sk2 else (None, None)
            ins = [lay(t) for t in (qr, kr, vr, k2r, v2r)]
            tol_rel, tol_abs = 2.0 ** -8, 2e-2
        qd, kd, vd, k2d, v2d = ins
        kall, vall = (kr, vr) if not Sk2 else (torch.cat([kr, k2r], 2), torch.cat([vr, v2r], 2))
        ro, rl = O.attn_fwd_ref(qr, kall, vall)
        o, l = ops.attn_fwd(qd, kd, vd, k2=k2d, v2=v2d, **kw)
        # outputs here are not averages over many keys and reach 3-4: the bound scales with them
        assert _err(o, ro) <= max(tol_abs, tol_rel * ro.abs().max().item()) and _err(l, rl) <= 1e-3, what
        plan = ops.launch_plan(qd, kd, k2=k2d)
        seen["balanced"] += plan["ranges"] > 0
        if not tune["streamed"]:
            o2, l2 = ops.attn_fwd(qd, kd, vd, k2=k2d, v2=v2d, **kw)
            assert torch.equal(o, o2) and torch.equal(l, l2), what
            if 0 < plan["workspace_bytes"] <= 32 * 1024 * 1024:
                o3, l3 = torch.full_like(o, float("nan")), torch.full_like(l, float("nan"))
                ops.attn_fwd(qd, kd, vd, k2=k2d, v2=v2d, out=o3, lse=l3, noalloc=True, **kw)
                assert torch.equal(o, o3) and torch.equal(l, l3), what
        # ring: the block of (k, v) alone, then this call's keys folded on top
        acc_o = torch.full((B, H, Sq, D), float("nan"), device=gpu)
        acc_l = torch.full((B, H, Sq), float("nan"), device=gpu)
        ref_o, ref_l = torch.empty_like(acc_o), torch.empty_like(acc_l)
        fin = torch.empty(B, H, Sq, D, dtype=dtype, device=gpu)
        ref_fin = torch.empty_like(fin)
        ops.attn_fwd_accumulate(qd, kd, vd, acc_o, acc_l, first=True, **kw)
        bo, bl = ops.attn_fwd(qd, kd, vd, **kw)
        ops.lse_merge(ref_o, ref_l, bo, bl, first=True)
        ops.attn_fwd_accumulate(qd, kd, vd, acc_o, acc_l, final_out=fin, k2=k2d, v2=v2d, **kw)
        ops.lse_merge(ref_o, ref_l, o, l, final_out=ref_fin)
        r1o, r1l = O.attn_fwd_ref(qr, kr, vr)
        mo, ml = O.merge_ref(r1o.to(dtype).double(), r1l, ro.to(dtype), rl)
        assert _err(fin, mo) <= max(tol_abs, 2 * tol_rel * mo.abs().max().item()) and _err(acc_l, ml) <= 1e-3, what
        ring_plans = [ops.launch_plan(qd, kd, k2=x, ring_step=True) for x in (None, k2d)]
        seen["ring_balanced"] += ring_plans[1]["ranges"] > 0
        same_cut = all((a["ranges"] == 0 and b["ranges"] == 0) or
                       all(a[f] == b[f] for f in ("rows_per_workgroup", "ranges", "range_len", "whole_tiles", "claimers"))
                       for a, b in zip([ops.launch_plan(qd, kd, k2=x) for x in (None, k2d)], ring_plans))
        if not tune["streamed"] and same_cut:
            assert torch.equal(fin, ref_fin) and torch.equal(acc_l, ref_l) and torch.equal(acc_o, ref_o), what
    assert seen["balanced"] + seen["ring_balanced"] > 0, seen   # the seeds do reach balanced launches


# ---------------------------------------------------------------------------- fused ring step
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float16, 128), (torch.bfloat16, 64),
                                      (torch.bfloat16, 72), (torch.float16, 104), (torch.float16, 24)])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_fused_ring_step_equals_forward_plus_merge(gpu, force_rows, dtype, D, layout):
    """xdit_attn_fwd_accumulate = xdit_attn_fwd + xdit_lse_merge, bit for bit, over three steps
    (initialise, fold, fold with the final cast), in both memory layouts, with the ragged sizes
    and every workgroup shape; against the oracle's fold as well."""
    B, H, Sq = 2, 3, 333
    g = torch.Generator().manual_seed(D + Sq)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    chunks = [(torch.randn(B, H, n, D, generator=g).to(dtype), torch.randn(B, H, n, D, generator=g).to(dtype)) for n in (257, 64, 130)]
    for rows in (128, 256, 384):
        force_rows(rows)
        qd = _layout(q, layout, gpu)
        acc_o = _layout(torch.full((B, H, Sq, D), float("nan")), layout, gpu)
        acc_l = torch.full((B, Sq, H, 1), float("nan"), device=gpu).squeeze(-1).transpose(1, 2)  # legacy (B,S,H,1) layout
        ref_o = torch.empty(B, H, Sq, D, device=gpu)
        ref_l = torch.empty(B, H, Sq, device=gpu)
        fin = torch.empty(B, H, Sq, D, dtype=dtype, device=gpu)
        ref_fin = torch.empty_like(fin)
        oo = ol = None
        for i, (k, v) in enumerate(chunks):
            kd, vd = _layout(k, layout, gpu), _layout(v, layout, gpu)
            last = i + 1 == len(chunks)
            ops.attn_fwd_accumulate(qd, kd, vd, acc_o, acc_l, first=i == 0, final_out=fin if last else None)
            bo, bl = ops.attn_fwd(qd, kd, vd)
            ops.lse_merge(ref_o, ref_l, bo, bl, first=i == 0, final_out=ref_fin if last else None)
            assert torch.equal(acc_o, ref_o) and torch.equal(acc_l, ref_l), (rows, i)
            ro, rl = O.attn_fwd_ref(q, k, v)
            oo, ol = (ro.to(dtype).double(), rl) if oo is None else O.merge_ref(oo, ol, ro.to(dtype), rl)
        assert torch.equal(fin, ref_fin)
        assert _err(acc_o, oo) <= 2e-2 and _err(acc_l, ol) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("cus", [1, 0])
@pytest.mark.parametrize("D", [72, 128, 16])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_fused_ring_step_fp32_equals_forward_plus_merge(gpu, monkeypatch, cus, D, layout):
    """The fp32 ring step (both workgroup forms of the fp32 kernel) against forward + merge, bit
    for bit, and against the oracle's fold."""
    monkeypatch.setitem(ops.TUNING, "cu_count", cus)
    B, H, Sq = 2, 2, 150
    g = torch.Generator().manual_seed(D + 7)
    q = torch.randn(B, H, Sq, D, generator=g)
    chunks = [(torch.randn(B, H, n, D, generator=g), torch.randn(B, H, n, D, generator=g)) for n in (97, 32, 130)]
    qd = _layout(q, layout, gpu)
    acc_o = _layout(torch.full((B, H, Sq, D), float("nan")), layout, gpu)
    acc_l = torch.full((B, Sq, H, 1), float("nan"), device=gpu).squeeze(-1).transpose(1, 2)
    ref_o, ref_l = torch.empty(B, H, Sq, D, device=gpu), torch.empty(B, H, Sq, device=gpu)
    fin = torch.empty(B, H, Sq, D, device=gpu)
    oo = ol = None
    for i, (k, v) in enumerate(chunks):
        kd, vd = _layout(k, layout, gpu), _layout(v, layout, gpu)
        last = i + 1 == len(chunks)
        ops.attn_fwd_accumulate(qd, kd, vd, acc_o, acc_l, first=i == 0, final_out=fin if last else None)
        bo, bl = ops.attn_fwd(qd, kd, vd)
        ops.lse_merge(ref_o, ref_l, bo, bl, first=i == 0)
        assert torch.equal(acc_o, ref_o) and torch.equal(acc_l, ref_l), i
        ro, rl = O.attn_fwd_ref(q, k, v)
        oo, ol = (ro, rl) if oo is None else O.merge_ref(oo, ol, ro, rl)
    assert torch.equal(fin, ref_o)
    assert _err(acc_o, oo) <= 2e-5 and _err(acc_l, ol) <= 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_fused_ring_step_fp8_equals_forward_plus_merge(gpu, force_rows, out_dtype, layout):
    """The fp8 ring step in every workgroup shape against forward + merge, bit for bit, with a
    second KV segment on one step; and against the oracle's fold of the dequantised inputs."""
    B, H, Sq, D = 1, 3, 333, 128
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, H, Sq, D, generator=g)
    chunks = [(torch.randn(B, H, n, D, generator=g), torch.randn(B, H, n, D, generator=g)) for n in (257, 64, 130)]
    jk, jv = torch.randn(B, H, 50, D, generator=g), torch.randn(B, H, 50, D, generator=g)
    q8, qs = ops.fp8_quant(q.to(gpu))
    q8l = _layout(q8.cpu().view(torch.uint8), layout, gpu).view(torch.float8_e4m3fn)
    quant = []
    for k, v in chunks:
        k8, j8, ks = ops.fp8_quant(k.to(gpu), x2=jk.to(gpu))
        v8, w8, vs = ops.fp8_quant(v.to(gpu), x2=jv.to(gpu))
        quant.append((k8, v8, j8, w8, ks, vs))
    for rows in (128, 256, 384):
        force_rows(rows)
        acc_o = _layout(torch.full((B, H, Sq, D), float("nan")), layout, gpu)
        acc_l = torch.full((B, Sq, H, 1), float("nan"), device=gpu).squeeze(-1).transpose(1, 2)
        ref_o, ref_l = torch.empty(B, H, Sq, D, device=gpu), torch.empty(B, H, Sq, device=gpu)
        fin = torch.empty(B, H, Sq, D, dtype=out_dtype, device=gpu)
        ref_fin = torch.empty_like(fin)
        oo = ol = None
        for i, (k8, v8, j8, w8, ks, vs) in enumerate(quant):
            last = i + 1 == len(quant)
            kw = dict(q_descale=qs, k_descale=ks, v_descale=vs, out_dtype=out_dtype)
            if i == 1:
                kw.update(k2=j8, v2=w8)
            ops.attn_fwd_accumulate(q8l, k8, v8, acc_o, acc_l, first=i == 0, final_out=fin if last else None, **kw)
            bo, bl = ops.attn_fwd(q8l, k8, v8, **kw)
            ops.lse_merge(ref_o, ref_l, bo, bl, first=i == 0, final_out=ref_fin if last else None)
            assert torch.equal(acc_o, ref_o) and torch.equal(acc_l, ref_l), (rows, i)
            kd, vd = O.dequant(k8.cpu(), ks.cpu()), O.dequant(v8.cpu(), vs.cpu())
            if i == 1:
                kd, vd = torch.cat([kd, O.dequant(j8.cpu(), ks.cpu())], 2), torch.cat([vd, O.dequant(w8.cpu(), vs.cpu())], 2)
            ro, rl = O.attn_fwd_ref(O.dequant(q8.cpu(), qs.cpu()), kd, vd)
            oo, ol = (ro.to(out_dtype).double(), rl) if oo is None else O.merge_ref(oo, ol, ro.to(out_dtype), rl)
        assert torch.equal(fin, ref_fin)
        assert _err(acc_o, oo) <= 6e-2 and _err(acc_l, ol) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("kind,rows,H,Sq,Sk,parts_first,counter", [
    ("bf16", 256, 3, 4608, 1152, 0, 0),      # every tile shared, parts of a tile end together: whoever completes it folds it
    ("bf16", 256, 24, 4608, 4608, 1, 0),     # whole tiles too, one range per claimer: parts first, slices folded at the ends
    ("bf16", 128, 24, 4608, 4608, 1, 0),
    ("fp16", 256, 24, 4608, 3072, 1, 0),
    ("bf16-d64", 256, 24, 4608, 4608, 1, 0),
    ("bf16-d72", 128, 24, 4608, 4608, 1, 0),
    ("bf16", 256, 12, 8192, 16384, 0, 1),    # long shares: ranges handed out through the counter
    ("fp8", 256, 24, 4608, 4608, 1, 0),
    ("fp8", 128, 24, 4608, 4608, 1, 0),
])
def test_balanced_fused_ring_step_equals_balanced_forward_plus_merge(gpu, monkeypatch, kind, rows, H, Sq, Sk, parts_first, counter):
    """The ring step with a workspace: the shared query tiles of the last round go through the
    workspace and are folded, and folded on into the accumulator, by the attention kernel's own
    workgroups (fold duties).  Three steps (initialise; fold, with a joint KV segment; fold with
    the final cast) must equal xdit_attn_fwd with the same launch geometry + xdit_lse_merge bit
    for bit, twice in a row on the same workspace (its counters return to zero), and the oracle's
    fold on probe rows."""
    monkeypatch.setitem(ops.TUNING, "rows_per_workgroup", rows)
    monkeypatch.setitem(ops.TUNING, "balance", 2)
    monkeypatch.setitem(ops.TUNING, "streamed", 0)   # bit equality: the fixed work geometry on both sides
    D = {"bf16-d64": 64, "bf16-d72": 72}.get(kind, 128)
    dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    g = torch.Generator(device=gpu).manual_seed(H + Sk)
    mk = lambda n: torch.randn(1, H, n, D, generator=g, device=gpu)
    q = mk(Sq)
    chunks = [(mk(Sk), mk(Sk)) for _ in range(3)]
    jk, jv = mk(77), mk(77)
    if kind == "fp8":
        q_in, qs = ops.fp8_quant(q)
        steps = []
        for i, (k, v) in enumerate(chunks):
            k8, j8, ks = ops.fp8_quant(k, x2=jk)
            v8, w8, vs = ops.fp8_quant(v, x2=jv)
            kw = dict(q_descale=qs, k_descale=ks, v_descale=vs, out_dtype=dtype)
            if i == 1:
                kw.update(k2=j8, v2=w8)
            steps.append((k8, v8, kw))
        ref_in = lambda t, s: O.dequant(t.cpu(), s.cpu())
    else:
        q_in = q.to(dtype)
        steps = [(k.to(dtype), v.to(dtype), dict(k2=jk.to(dtype), v2=jv.to(dtype)) if i == 1 else {}) for i, (k, v) in enumerate(chunks)]
    plan = ops.launch_plan(q_in, steps[0][0], ring_step=True)
    assert plan["ranges"] > 0 and plan["fold_in_kernel"] == 1 and plan["parts_first"] == parts_first and plan["counter"] == counter, plan
    assert ops.launch_plan(q_in, steps[0][0])["ranges"] == plan["ranges"]   # the plain forward is cut the same way
    results = []
    for repeat in range(2):
        acc_o = torch.full((1, H, Sq, D), float("nan"), device=gpu)
        acc_l = torch.full((1, H, Sq), float("nan"), device=gpu)
        ref_o, ref_l = torch.empty_like(acc_o), torch.empty_like(acc_l)
        fin = torch.empty(1, H, Sq, D, dtype=dtype, device=gpu)
        ref_fin = torch.empty_like(fin)
        for i, (k, v, kw) in enumerate(steps):
            last = i + 1 == len(steps)
            ops.attn_fwd_accumulate(q_in, k, v, acc_o, acc_l, first=i == 0, final_out=fin if last else None, **kw)
            bo, bl = ops.attn_fwd(q_in, k, v, **kw)
            ops.lse_merge(ref_o, ref_l, bo, bl, first=i == 0, final_out=ref_fin if last else None)
            assert torch.equal(acc_o, ref_o) and torch.equal(acc_l, ref_l), (repeat, i)
        assert torch.equal(fin, ref_fin)
        results.append((acc_o, acc_l, fin))
    assert all(torch.equal(a, b) for a, b in zip(*results))
    # values: probe rows of the whole fold against the oracle
    probe = torch.arange(0, Sq, 509)
    oo = ol = None
    for i, (k, v, kw) in enumerate(steps):
        if kind == "fp8":
            kd, vd = ref_in(k, kw["k_descale"]), ref_in(v, kw["v_descale"])
            if i == 1:
                kd, vd = torch.cat([kd, ref_in(kw["k2"], kw["k_descale"])], 2), torch.cat([vd, ref_in(kw["v2"], kw["v_descale"])], 2)
            qd = ref_in(q_in, qs)
        else:
            kd, vd = k.cpu(), v.cpu()
            if i == 1:
                kd, vd = torch.cat([kd, kw["k2"].cpu()], 2), torch.cat([vd, kw["v2"].cpu()], 2)
            qd = q_in.cpu()
        ro, rl = O.attn_fwd_ref(qd[:, :, probe], kd, vd)
        oo, ol = (ro.to(dtype).double(), rl) if oo is None else O.merge_ref(oo, ol, ro.to(dtype), rl)
    tol = 6e-2 if kind == "fp8" else 2e-2
    assert _err(results[0][0][:, :, probe.to(gpu)], oo) <= tol and _err(results[0][1][:, :, probe.to(gpu)], ol) <= 1e-3


@pytest.mark.gpu
def test_fused_ring_step_last_step_may_skip_the_accumulator(gpu):
    B, H, Sq, D = 1, 2, 200, 128
    q, k, v = (torch.randn(B, H, n, D).bfloat16().to(gpu) for n in (Sq, 300, 300))
    acc_o = torch.randn(B, H, Sq, D, device=gpu)
    acc_l = torch.randn(B, H, Sq, device=gpu)
    a2, l2 = acc_o.clone(), acc_l.clone()
    fin, fin2 = torch.empty(B, H, Sq, D, dtype=torch.bfloat16, device=gpu), torch.empty(B, H, Sq, D, dtype=torch.bfloat16, device=gpu)
    ops.attn_fwd_accumulate(q, k, v, acc_o, acc_l, final_out=fin)
    before = a2.clone()
    ops.attn_fwd_accumulate(q, k, v, a2, l2, final_out=fin2, discard_acc_out=True)
    assert torch.equal(fin, fin2) and torch.equal(acc_l, l2)
    assert torch.equal(a2, before) and torch.equal(fin, acc_o.bfloat16())
    with pytest.raises(ValueError):
        ops.attn_fwd_accumulate(q, k, v, a2, l2, discard_acc_out=True)


@pytest.mark.gpu
@pytest.mark.parametrize("strategy", [None, "front", "rear"])
def test_ring_loop_fused_equals_two_call_loop(gpu, monkeypatch, strategy):
    """The BSHD ring loop takes the fused step where it can; forcing the kernel call +
    update_out_and_lse sequence instead must give the same bits."""
    B, S, H, D, P = 1, 4 * 300, 4, 128, 4
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(B, S, H, D, generator=g).bfloat16().to(gpu) for _ in range(3))
    kw = {}
    if strategy:
        kw = dict(joint_tensor_key=torch.randn(B, 77, H, D, generator=g).bfloat16().to(gpu),
                  joint_tensor_value=torch.randn(B, 77, H, D, generator=g).bfloat16().to(gpu), joint_strategy=strategy)
    o1, l1, _ = ring.xdit_ring_flash_attn_func(q, k, v, return_attn_probs=True, group=ring.LocalRing(P, rank=1), **kw)
    monkeypatch.setattr(ops, "fused_ring_step_supported", lambda q: False)
    o2, l2, _ = ring.xdit_ring_flash_attn_func(q, k, v, return_attn_probs=True, group=ring.LocalRing(P, rank=1), **kw)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    kall = k if not strategy else torch.cat([k, kw["joint_tensor_key"]], 1)
    vall = v if not strategy else torch.cat([v, kw["joint_tensor_value"]], 1)
    ro, rl = O.attn_fwd_ref(*(t.transpose(1, 2).cpu() for t in (q, kall, vall)))
    assert _err(o1.transpose(1, 2), ro) <= 2e-2 and _err(l1, rl) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("strategy", [None, "front", "rear"])
def test_usp_ring_fused_equals_merger_loop(gpu, monkeypatch, strategy):
    """usp.ring_attn takes the fused step for our 16-bit backend (the launch count shows it); the
    attention-function + SDPAMerger loop must give the same bits."""
    g = torch.Generator().manual_seed(31)
    q, k, v = (torch.randn(1, 4, 4 * 200, 128, generator=g).bfloat16().to(gpu) for _ in range(3))
    jk = jv = None
    mk = lambda: None
    if strategy:
        jk, jv = (torch.randn(1, 4, 50, 128, generator=g).bfloat16().to(gpu) for _ in range(2))
        mk = lambda: dict(joint_key=jk, joint_value=jv, joint_strategy=strategy, step=0, total_steps=4)
    fn = usp._get_attention_function()
    calls = []
    real = ops.attn_fwd_accumulate
    monkeypatch.setattr(ops, "attn_fwd_accumulate", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    a = usp.ring_attn(fn, q, k, v, ring_chunks=4, joint_attn_kwargs=mk())
    assert len(calls) == 4
    monkeypatch.setattr(ops, "fused_ring_step_supported", lambda q: False)
    b = usp.ring_attn(fn, q, k, v, ring_chunks=4, joint_attn_kwargs=mk())
    assert len(calls) == 4 and torch.equal(a, b)
    kall = k if not strategy else torch.cat([jk, k] if strategy == "front" else [k, jk], 2)
    vall = v if not strategy else torch.cat([jv, v] if strategy == "front" else [v, jv], 2)
    ro, _ = O.attn_fwd_ref(q.cpu(), kall.cpu(), vall.cpu())
    assert _err(a, ro) <= 2e-2


# ---------------------------------------------------------------------------- quantiser
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fp8_quant_bit_exact(gpu, dtype):
    g = torch.Generator().manual_seed(8)
    x = (torch.randn(2, 3, 333, 128, generator=g) * torch.arange(1, 7).reshape(2, 3, 1, 1)).to(dtype)
    y, d = ops.fp8_quant(_layout(x, "bshd", gpu))
    ry, rd = O.per_head_quant_ref(x)
    assert torch.equal(y.cpu().view(torch.uint8), ry.view(torch.uint8)) and torch.equal(d.cpu(), rd)
    y, d = AB.per_tensor_quant(x.to(gpu))
    ry, rd = O.per_tensor_quant_ref(x)
    assert torch.equal(y.cpu().view(torch.uint8), ry.view(torch.uint8)) and torch.equal(d.cpu(), rd.contiguous())
    s = torch.tensor(0.05)
    y, d = AB.per_tensor_quant(x.to(gpu), scale=s.to(gpu))
    ry, rd = O.per_tensor_quant_ref(x.clamp(-448 * 0.05, 448 * 0.05), scale=s)
    assert torch.equal(y.cpu().view(torch.uint8), ry.view(torch.uint8)) and torch.all(d.cpu() == 0.05)
    y0, d0 = ops.fp8_quant(torch.zeros(1, 1, 8, 128, device=gpu))
    assert d0.item() == 1.0 and torch.all(y0.float() == 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("block,D", [(128, 128), (32, 128), (8, 64), (2, 128), (64, 64), (16, 96)])
def test_fp8_quant_with_hadamard_rotation(gpu, dtype, block, D):
    """Rotation fused into the quantiser against rotate-then-quantise on the oracle.  The kernel
    sums the +-x terms in fp32 in butterfly order, the oracle in float64, so a value that lands
    within fp32 rounding of a rounding boundary of `dtype` (and then of fp8) may differ by one
    step: at most 1 % of the bytes may differ and then only by one fp8 step; scales may differ by
    one step of `dtype`."""
    g = torch.Generator().manual_seed(block + D)
    x = torch.randn(2, 3, 77, D, generator=g)
    x[0, 1, 5, 3] = 40.0  # an outlier
    x = x.to(dtype)
    y, d = ops.fp8_quant(_layout(x, "bshd", gpu), hadamard_block=block)
    rot = O.hadamard_rotate_ref(x, block)
    ry, rd = O.per_head_quant_ref(rot)
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -22}[dtype]
    assert torch.allclose(d.cpu(), rd, rtol=2 * eps, atol=0)
    a, b = y.cpu().view(torch.uint8).int(), ry.view(torch.uint8).int()
    assert (a != b).float().mean().item() <= 0.01
    assert ((a - b).abs() <= 1).all()
    # rotating back (R is symmetric and orthonormal) recovers x to fp8 accuracy
    back = O.hadamard_rotate_ref(O.dequant(y.cpu(), d.cpu()).double(), block)
    assert (back - x.double()).abs().max().item() <= 2.0 ** -4 * x.double().abs().max().item()
    with pytest.raises(ValueError):
        ops.fp8_quant(x.to(gpu), hadamard_block=48)
    with pytest.raises(ValueError):
        ops.fp8_quant(x.to(gpu), hadamard_block=256)


@pytest.mark.parametrize("outlier", [1.0, 12.0])
def test_fp8_adapter_rotation(gpu, outlier):
    """The fp8 adapter with q and k rotated inside the quantiser (q.k is invariant under a common
    rotation) against the attention of the UNQUANTISED inputs.  Without outliers both forms stay
    within the fp8 tolerance; with one channel of q and k 12x larger (which per-tensor fp8
    quantisation resolves badly) the rotation must cut the error by more than half."""
    q, k, v = O.make_qkv(1, 4, 640, 128, seed=71, dtype=torch.float32)
    q[..., 7] *= outlier
    k[..., 7] *= outlier
    s = 1.0 if outlier == 1.0 else 0.3
    q, k, v = (t.to(torch.bfloat16) for t in (q * s, k * s, v))
    ro, rl = O.attn_fwd_ref(q, k, v)
    fn = AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355_FP8]
    o_rot, l_rot = fn(q.to(gpu), k.to(gpu), v.to(gpu), 0.0, False)
    o_off, l_off = fn(q.to(gpu), k.to(gpu), v.to(gpu), 0.0, False, attention_kwargs={"hadamard_block": 0})
    assert AB.FP8_HADAMARD_BLOCK == 128 and not torch.equal(o_rot, o_off)
    if outlier == 1.0:
        assert _err(o_rot, ro) <= 6e-2 and _err(o_off, ro) <= 6e-2
        assert _err(l_rot, rl) <= 5e-2 and _err(l_off, rl) <= 5e-2
    else:
        assert _err(o_rot, ro) <= 0.5 * _err(o_off, ro) and _err(l_rot, rl) <= 0.5 * _err(l_off, rl)


# ---------------------------------------------------------------------------- call surfaces
@pytest.mark.parametrize("strategy", ["front", "rear"])
@pytest.mark.parametrize("chunks", [1, 2])
def test_usp_joint_vs_oracle(gpu, strategy, chunks):
    q, k, v = O.make_qkv(1, 4, 512, 128, seed=31, rmsnorm=True, dtype=torch.bfloat16)
    jq, jk, jv = O.make_qkv(1, 4, 77, 128, seed=32, rmsnorm=True, dtype=torch.bfloat16)
    cat = (lambda a, b: torch.cat([a, b], 2)) if strategy == "rear" else (lambda a, b: torch.cat([b, a], 2))
    ro, _ = O.attn_fwd_ref(cat(q, jq), cat(k, jk), cat(v, jv))
    o = usp.USP(q.to(gpu), k.to(gpu), v.to(gpu), joint_query=jq.to(gpu), joint_key=jk.to(gpu), joint_value=jv.to(gpu),
                joint_strategy=strategy, ring_chunks=chunks)
    assert o.shape == (1, 4, 589, 128) and _err(o, ro) <= 2e-2


@pytest.mark.parametrize("strategy", ["front", "rear"])
def test_long_context_layer_joint_vs_oracle(gpu, strategy):
    """The layer form in BSHD with fp16, tolerance of the reference's own layer test (1e-2)."""
    q, k, v = O.make_qkv(1, 4, 256, 128, seed=41, dtype=torch.float16)
    jq, jk, jv = O.make_qkv(1, 4, 64, 128, seed=42, dtype=torch.float16)
    cat = (lambda a, b: torch.cat([a, b], 2)) if strategy == "rear" else (lambda a, b: torch.cat([b, a], 2))
    ro, _ = O.attn_fwd_ref(cat(q, jq), cat(k, jk), cat(v, jv))
    b = lambda t: t.transpose(1, 2).contiguous().to(gpu)
    layer = ring.xFuserLongContextAttention(ring_group=ring.LocalRing(2))
    o = layer(None, b(q), b(k), b(v), joint_tensor_query=b(jq), joint_tensor_key=b(jk), joint_tensor_value=b(jv),
              joint_strategy=strategy)
    assert o.shape == (1, 320, 4, 128) and _err(o.transpose(1, 2), ro) <= 1e-2


def test_fp8_backend_adapter(gpu):
    q, k, v = O.make_qkv(1, 4, 512, 128, seed=51, dtype=torch.bfloat16)
    ro, rl = O.attn_fwd_ref(q, k, v)
    o, l = AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355_FP8](q.to(gpu), k.to(gpu), v.to(gpu), 0.0, False)
    assert o.dtype == torch.bfloat16 and _err(o, ro) <= 6e-2 and _err(l, rl) <= 5e-2  # vs the UNQUANTISED inputs
    assert torch.equal(o, usp.attention(q.to(gpu), k.to(gpu), v.to(gpu), backend=AB.AttentionBackendType.MI355_FP8))


@pytest.mark.parametrize("strategy", ["rear", "front"])
def test_fp8_backend_adapter_joint_keys_without_a_copy(gpu, monkeypatch, strategy):
    """The fp8 adapter with joint (text) keys/values: they are quantised with the scale of the
    keys/values they are attended with (one abs-max over both) and handed to the kernel as its
    second KV segment.  Bytes and scales must equal what quantising the concatenation gives (the
    reference's order of operations: usp.py:239-241, then per_tensor_quant), no torch.cat of K or
    V may run, and the output must match the oracle's attention of the dequantised tensors."""
    q, k, v = O.make_qkv(1, 3, 400, 128, seed=71, dtype=torch.bfloat16)
    _, jk, jv = O.make_qkv(1, 3, 77, 128, seed=72, dtype=torch.bfloat16)
    jk = jk * 1.5  # the joint keys carry the abs-max
    order = (lambda a, b: torch.cat([a, b], 2)) if strategy == "rear" else (lambda a, b: torch.cat([b, a], 2))
    k8, j8, kd = AB.per_tensor_quant(k.to(gpu), x2=jk.to(gpu))
    rk8, rkd = O.per_tensor_quant_ref(torch.cat([k, jk], 2))
    assert torch.equal(torch.cat([k8, j8], 2).cpu().view(torch.uint8), rk8.view(torch.uint8)) and torch.equal(kd.cpu(), rkd.contiguous())
    # reference of the whole call: quantise q, cat(k), cat(v) per tensor, attend the dequantised tensors
    (q8, qd), (kk8, kkd), (vv8, vvd) = (O.per_tensor_quant_ref(t) for t in (q, order(k, jk), order(v, jv)))
    ro, rl = O.attn_fwd_ref(O.dequant(q8, qd), O.dequant(kk8, kkd), O.dequant(vv8, vvd))
    cats = []
    real_cat = torch.cat
    monkeypatch.setattr(torch, "cat", lambda *a, **kw: (cats.append(1), real_cat(*a, **kw))[1])
    fn = AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355_FP8]
    o, l = fn(q.to(gpu), k.to(gpu), v.to(gpu), 0.0, False, attention_kwargs={"hadamard_block": 0},
              joint_kv=(jk.to(gpu), jv.to(gpu), strategy))
    monkeypatch.undo()
    assert not cats
    # (keys wider than unit RMS concentrate the softmax on few keys, the hard case for an fp8 P:
    # the bar is applied relative to the largest output where that exceeds 1)
    assert _err(o, ro) <= 6e-2 * max(1.0, ro.abs().max().item()) and _err(l, rl) <= 1e-3
    # through USP, with the rotation on (the default): the same call as the adapter's, and close to
    # the attention of the unquantised tensors (which also sees the fp8 rounding of q, k and v)
    uo = usp.USP(q[:, :, :300].to(gpu), k.to(gpu), v.to(gpu), joint_query=q[:, :, 300:].to(gpu), joint_key=jk.to(gpu),
                 joint_value=jv.to(gpu), joint_strategy=strategy, backend=AB.AttentionBackendType.MI355_FP8)
    qq = order(q[:, :, :300], q[:, :, 300:])
    direct, _ = fn(qq.to(gpu), k.to(gpu), v.to(gpu), 0.0, False, joint_kv=(jk.to(gpu), jv.to(gpu), strategy))
    assert torch.equal(uo, direct)
    fo, _ = O.attn_fwd_ref(qq, order(k, jk), order(v, jv))
    assert _err(uo, fo) <= 0.25


def test_fp8_backend_adapter_static_scale(gpu, monkeypatch):
    """A static scale for q, k and v (the reference takes one from
    XFUSER_AITER_FP8_STATIC_SCALE_WITH_DESCALE, attention_backend.py:735-745): per call through
    attention_kwargs or as the module's default; descales then equal the scale."""
    q, k, v = O.make_qkv(1, 2, 256, 128, seed=81, dtype=torch.bfloat16)
    s = 0.02
    (q8, qd), (k8, kd), (v8, vd) = (O.per_tensor_quant_ref(t.clamp(-448 * s, 448 * s), scale=torch.tensor(s)) for t in (q, k, v))
    ro, rl = O.attn_fwd_ref(O.dequant(q8, qd), O.dequant(k8, kd), O.dequant(v8, vd))
    fn = AB.ATTENTION_FUNCTION_REGISTRY[AB.AttentionBackendType.MI355_FP8]
    o, l = fn(q.to(gpu), k.to(gpu), v.to(gpu), 0.0, False, attention_kwargs={"hadamard_block": 0, "fp8_static_scale": s})
    assert _err(o, ro) <= 6e-2 and _err(l, rl) <= 1e-3
    monkeypatch.setattr(AB, "FP8_STATIC_SCALE", s)
    o2, l2 = fn(q.to(gpu), k.to(gpu), v.to(gpu), 0.0, False, attention_kwargs={"hadamard_block": 0})
    assert torch.equal(o, o2) and torch.equal(l, l2)


def test_fp8_quant_with_and_without_scratch(gpu):
    """The quantiser through the C ABI with no scratch buffer (four launches, atomics on the descale
    buffer) and with one (two launches): the same bytes and descales, per head and per tensor, with
    a second tensor sharing the scales."""
    import ctypes
    from xdit_amd import _lib
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(2, 3, 301, 128, generator=g) * torch.arange(1, 7).reshape(2, 3, 1, 1)).bfloat16().to(gpu)
    x2 = (torch.randn(2, 3, 40, 128, generator=g) * 9).bfloat16().to(gpu)
    for per_tensor in (False, True):
        want = ops.fp8_quant(x, per_tensor=per_tensor, x2=x2)
        ry, rd = (O.per_tensor_quant_ref if per_tensor else O.per_head_quant_ref)(torch.cat([x, x2], 2).cpu())
        assert torch.equal(torch.cat(want[:2], 2).cpu().view(torch.uint8), ry.view(torch.uint8)) and torch.equal(want[2].cpu(), rd.contiguous())
        y = torch.empty_like(want[0]); y2 = torch.empty_like(want[1]); d = torch.empty_like(want[2])
        a = _lib.QuantArgs()
        a.struct_size = ctypes.sizeof(_lib.QuantArgs)
        a.in_dtype, a.per_tensor = _lib.DTYPE_BF16, int(per_tensor)
        a.B, a.H, a.D, a.S, a.S2 = 2, 3, 128, 301, 40
        a.x, a.y, a.descale, a.x2, a.y2 = x.data_ptr(), y.data_ptr(), d.data_ptr(), x2.data_ptr(), y2.data_ptr()
        a.x_stride, a.y_stride = ops._strides(x), ops._strides(y)
        a.x2_stride, a.y2_stride = ops._strides(x2), ops._strides(y2)
        a.stream = ops._stream(x.device)
        _lib.check(_lib.lib().xdit_fp8_quant(ctypes.byref(a)))   # scratch = NULL
        torch.cuda.synchronize()
        assert all(torch.equal(p.view(torch.uint8), r.view(torch.uint8)) for p, r in ((y, want[0]), (y2, want[1]))) and torch.equal(d, want[2])


def test_runs_on_the_callers_stream(gpu):
    """Launches go to the current stream: work queued on a side stream is ordered with it."""
    q, k, v = (torch.randn(1, 2, 512, 128, device=gpu).bfloat16() for _ in range(3))
    ref_o, ref_l = ops.attn_fwd(q, k, v)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        q2 = q * 1.0
        o, l = ops.attn_fwd(q2, k, v)
    s.synchronize()
    assert torch.equal(o, ref_o) and torch.equal(l, ref_l)


# ---------------------------------------------------------------------------- torch.library ops
def test_custom_ops_opcheck_and_compile(gpu):
    """The registered ops pass torch's own consistency checks (schema, fake vs real outputs,
    functionalisation of the in-place merge) and a compiled caller gives the eager bits without a
    graph break."""
    from xdit_amd import custom_ops  # noqa: F401
    q, k, v = O.make_qkv(1, 2, 300, 128, seed=61, dtype=torch.bfloat16)
    jk, jv = (t[:, :, :40].contiguous() for t in O.make_qkv(1, 2, 64, 128, seed=62, dtype=torch.bfloat16)[1:])
    q, k, v, jk, jv = (t.to(gpu) for t in (q, k, v, jk, jv))
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(torch.ops.xdit_amd.attn_fwd.default, (q, k, v, 128 ** -0.5), test_utils=tests)
    torch.library.opcheck(torch.ops.xdit_amd.attn_fwd_joint.default, (q, k, v, jk, jv, 128 ** -0.5), test_utils=tests)
    torch.library.opcheck(torch.ops.xdit_amd.fp8_quant.default, (q, True, 128), test_utils=tests)
    o, l = ops.attn_fwd(q, k, v)
    acc_o, acc_l = o.float(), l.clone()
    torch.library.opcheck(torch.ops.xdit_amd.lse_merge.default, (acc_o, acc_l, o, l, False), test_utils=tests)

    eager = AB._mi355_attn_call(q, k, v, 0.0, False, joint_kv=(jk, jv, "rear"))

    def block(q, k, v, jk, jv):
        out, lse = AB._mi355_attn_call(q * 1, k, v, 0.0, False, joint_kv=(jk, jv, "rear"))
        return out + 0, lse

    co, cl = torch.compile(block, backend="aot_eager", fullgraph=True)(q, k, v, jk, jv)
    assert torch.equal(co, eager[0]) and torch.equal(cl, eager[1])

    def fp8_block(q, k, v):
        return AB._mi355_fp8_attn_call(q, k, v, 0.0, False)

    e8 = fp8_block(q, k, v)
    c8 = torch.compile(fp8_block, backend="aot_eager", fullgraph=True)(q, k, v)
    assert torch.equal(c8[0], e8[0]) and torch.equal(c8[1], e8[1])


def test_custom_ops_ring_step_and_joint_fp8_under_compile(gpu, monkeypatch):
    """The ring step, the fp8 forward with a second KV segment and the quantiser with a second
    tensor / a static scale as registered ops: torch's consistency checks, and compiled callers
    (`torch.compile(fullgraph=True)` of `usp.USP` with joint tensors on the fp8 backend, with a
    static scale too, and of `usp.ring_attn` over four chunks with joint keys on the last step)
    give the eager bits without a graph break."""
    from xdit_amd import custom_ops  # noqa: F401
    q, k, v = O.make_qkv(1, 2, 512, 128, seed=63, dtype=torch.bfloat16)
    jq, jk, jv = (t[:, :, :40].contiguous() for t in O.make_qkv(1, 2, 64, 128, seed=64, dtype=torch.bfloat16))
    q, k, v, jq, jk, jv = (t.to(gpu) for t in (q, k, v, jq, jk, jv))
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    scale = torch.tensor([0.01], device=gpu)
    torch.library.opcheck(torch.ops.xdit_amd.fp8_quant_ex.default, (k, jk, None, True, 128), test_utils=tests)
    torch.library.opcheck(torch.ops.xdit_amd.fp8_quant_ex.default, (k, None, scale, True, 0), test_utils=tests)
    k8, j8, kd = ops.fp8_quant(k, per_tensor=True, x2=jk)
    v8, w8, vd = ops.fp8_quant(v, per_tensor=True, x2=jv)
    q8, qd = ops.fp8_quant(q, per_tensor=True)
    # (torch's schema check hashes the inputs with arithmetic that fp8 tensors do not have)
    torch.library.opcheck(torch.ops.xdit_amd.attn_fwd_fp8_joint.default, (q8, k8, v8, j8, w8, qd, kd, vd, 128 ** -0.5, False), test_utils=("test_faketensor", "test_autograd_registration"))
    acc_o = torch.zeros(1, 2, 512, 128, device=gpu)
    acc_l = torch.zeros(1, 2, 512, device=gpu)
    fin = torch.empty_like(q)
    torch.library.opcheck(torch.ops.xdit_amd.attn_fwd_accumulate.default, (q, k, v, jk, jv, acc_o, acc_l, None, True, False, 128 ** -0.5), test_utils=tests)
    torch.library.opcheck(torch.ops.xdit_amd.attn_fwd_accumulate.default, (q, k, v, None, None, acc_o, acc_l, fin, False, True, 128 ** -0.5), test_utils=tests)

    def usp_fp8(q, k, v, jq, jk, jv):
        return usp.USP(q, k, v, joint_query=jq, joint_key=jk, joint_value=jv, joint_strategy="rear",
                       backend=AB.AttentionBackendType.MI355_FP8)

    eager = usp_fp8(q, k, v, jq, jk, jv)
    assert torch.equal(torch.compile(usp_fp8, backend="aot_eager", fullgraph=True)(q, k, v, jq, jk, jv), eager)
    monkeypatch.setattr(AB, "FP8_STATIC_SCALE", 0.02)
    eager_static = usp_fp8(q, k, v, jq, jk, jv)
    assert not torch.equal(eager_static, eager)
    assert torch.equal(torch.compile(usp_fp8, backend="aot_eager", fullgraph=True)(q, k, v, jq, jk, jv), eager_static)

    def ring(q, k, v, jq, jk, jv):
        return usp.USP(q, k, v, joint_query=jq, joint_key=jk, joint_value=jv, joint_strategy="rear", ring_chunks=4)

    eager_ring = ring(q, k, v, jq, jk, jv)
    assert torch.equal(torch.compile(ring, backend="aot_eager", fullgraph=True)(q, k, v, jq, jk, jv), eager_ring)
    fn = usp._get_attention_function()

    def ring_only(q, k, v):
        return usp.ring_attn(fn, q, k, v, ring_chunks=4)

    assert torch.equal(torch.compile(ring_only, backend="aot_eager", fullgraph=True)(q, k, v), ring_only(q, k, v))


# ---------------------------------------------------------------------------- HIP graphs
def test_graph_capture_and_replay_of_the_ring(gpu):
    """The launch-bound ring of four chunks (4 attention launches + combine + 4 merge launches)
    captured once in a HIP graph and replayed: every replay must equal the eager result for the
    inputs in the static buffers at that time, with eager launches and synchronisations between
    the replays (the workspace and all temporaries live in the graph's memory pool)."""
    fn = usp._get_attention_function()
    q, k, v = O.make_qkv(1, 8, 1536, 128, seed=81, rmsnorm=True, dtype=torch.bfloat16)
    sq, sk, sv = q.to(gpu), k.to(gpu), v.to(gpu)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # warm-up off the default stream, as graph capture requires
        for _ in range(2):
            usp.ring_attn(fn, sq, sk, sv, ring_chunks=4)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sout = usp.ring_attn(fn, sq, sk, sv, ring_chunks=4)
    for seed in (82, 83, 84):
        q2, k2, v2 = O.make_qkv(1, 8, 1536, 128, seed=seed, rmsnorm=True, dtype=torch.bfloat16)
        sq.copy_(q2.to(gpu)); sk.copy_(k2.to(gpu)); sv.copy_(v2.to(gpu))
        graph.replay()
        torch.cuda.synchronize()
        replayed = sout.clone()
        eager = usp.ring_attn(fn, sq, sk, sv, ring_chunks=4)   # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager)
        ro, _ = O.attn_fwd_ref(q2, k2, v2)
        assert _err(replayed, ro) <= 2e-2


def _claimed_ranges_problem(gpu, seed):
    """bf16 problem whose last round is handed out through the range counter at 384 rows."""
    g = torch.Generator(device=gpu).manual_seed(seed)
    return tuple(torch.randn(1, 12, n, 128, generator=g, device=gpu).bfloat16() for n in (32 * 384, 256 * 64, 256 * 64))


def test_claimed_ranges_in_a_graph_and_on_two_streams(gpu, force_rows):
    """The range counter is cleared by a kernel of the launch sequence, so a captured launch can
    be replayed; and two streams running such launches at the same time each have their own
    workspace (and counter).  Every result must equal the plain eager call bit for bit."""
    force_rows(384)
    q, k, v = _claimed_ranges_problem(gpu, 5)
    want = ops.attn_fwd(q, k, v)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.attn_fwd(q, k, v)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = ops.attn_fwd(q, k, v)
    for i in range(3):
        got[0].zero_(); got[1].zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), i
        ops.attn_fwd(q, k, v)  # eager work between the replays
        torch.cuda.synchronize()
    # two streams at once, different inputs
    q2, k2, v2 = _claimed_ranges_problem(gpu, 6)
    want2 = ops.attn_fwd(q2, k2, v2)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for _ in range(3):
        with torch.cuda.stream(s1):
            a = ops.attn_fwd(q, k, v)
        with torch.cuda.stream(s2):
            b = ops.attn_fwd(q2, k2, v2)
        outs.append((a, b))
    torch.cuda.synchronize()
    for a, b in outs:
        assert torch.equal(a[0], want[0]) and torch.equal(a[1], want[1])
        assert torch.equal(b[0], want2[0]) and torch.equal(b[1], want2[1])
