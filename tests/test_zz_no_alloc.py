"""xdit_attn_fwd_noalloc — the entry point for callers that cannot allocate device memory — against
xdit_attn_fwd on the same inputs, through the C ABI.  Both run the same kernels with the same
launch geometry, so outputs and log-sum-exps must be bit-identical (the bar for index and
scheduling work); what differs is where the partial results of the balanced launch live: in a
fixed array inside the library instead of a workspace of the caller.  Two calls in a row share
that array, the second with a smaller input, then an fp8 call; a problem that needs more
scratch than the array holds must be refused before anything is launched."""
import pytest
import torch

from xdit_amd import _lib, ops

pytestmark = pytest.mark.gpu
LIMIT = 32 * 1024 * 1024


@pytest.fixture(autouse=True)
def fixed_geometry(monkeypatch):
    """The comparison below is bit for bit, so both calls run with the default, fixed work geometry
    (under streamed sharing two runs of ONE entry point already differ in last bits)."""
    monkeypatch.setitem(ops.TUNING, "streamed", 0)


def _pair(q, k, v, **kw):
    B, H, Sq, D = q.shape
    odt = torch.bfloat16 if q.dtype == torch.float8_e4m3fn else q.dtype
    plan = ops.launch_plan(q, k)
    assert plan["ranges"] > 0 and 0 < plan["workspace_bytes"] <= LIMIT, plan   # the scratch is really used
    ref_o, ref_l = ops.attn_fwd(q, k, v, **kw)
    out = torch.full((B, H, Sq, D), float("nan"), dtype=odt, device=q.device)
    lse = torch.full((B, H, Sq), float("nan"), dtype=torch.float32, device=q.device)
    o, l = ops.attn_fwd(q, k, v, out=out, lse=lse, noalloc=True, **kw)
    assert o.data_ptr() == out.data_ptr() and l.data_ptr() == lse.data_ptr()
    torch.cuda.synchronize()
    assert torch.equal(out, ref_o) and torch.equal(lse, ref_l)
    return out, lse


def test_noalloc_entry_point_equals_attn_fwd(gpu):
    g = torch.Generator(device=gpu).manual_seed(5)
    mk = lambda H, S: tuple(torch.randn(1, H, S, 128, generator=g, device=gpu).bfloat16() for _ in range(3))
    big = mk(24, 4608)       # Flux-1024: 32 of 288 query tiles shared, 28.75 MB of partial results
    small = mk(3, 4608)      # 108 query tiles of 128 rows, all of them shared among 486 ranges
    o1, l1 = _pair(*big)
    o2, l2 = _pair(*small)
    # the second call has not disturbed what the first returned, and a repeat gives the same bits
    o1b, l1b = _pair(*big)
    assert torch.equal(o1, o1b) and torch.equal(l1, l1b)
    # the fp8 kernel shares the same array
    (q8, qd), (k8, kd), (v8, vd) = (ops.fp8_quant(t) for t in small)
    _pair(q8, k8, v8, q_descale=qd, k_descale=kd, v_descale=vd)
    # streamed sharing through the same entry point: equal to rounding
    out = torch.empty_like(big[0])
    lse = torch.empty(1, 24, 4608, device=gpu)
    ops.attn_fwd(*big, out=out, lse=lse, noalloc=True, streamed=True)
    assert ops.launch_plan(big[0], big[1], streamed=True)["streamed"] == 1
    assert (out.float() - o1.float()).abs().max().item() <= 2.0 ** -7 * o1.float().abs().max().item()
    assert (lse - l1).abs().max().item() <= 1e-5
    # a sane value check on top of the equality: rows of the small problem against fp32 torch
    q, k, v = (t.float() for t in small)
    s = (q[:, :, :64] @ k.transpose(-1, -2)) * 128 ** -0.5
    assert (o2[:, :, :64].float() - torch.softmax(s, -1) @ v).abs().max().item() <= 2e-2
    assert (l2[:, :, :64] - torch.logsumexp(s, -1)).abs().max().item() <= 1e-3


def test_noalloc_refuses_what_does_not_fit(gpu):
    q = torch.zeros(1, 12, 32 * 384, 128, dtype=torch.bfloat16, device=gpu)
    k = torch.zeros(1, 12, 256 * 64, 128, dtype=torch.bfloat16, device=gpu)
    assert ops.launch_plan(q, k)["workspace_bytes"] > LIMIT
    out = torch.full_like(q, 7.0)
    lse = torch.zeros(1, 12, 32 * 384, device=gpu)
    with pytest.raises(ValueError, match="bytes of scratch"):
        ops.attn_fwd(q, k, k, out=out, lse=lse, noalloc=True)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())   # nothing was launched
    # the same problem as a plain launch (the tuning field balance = 1) needs no scratch
    ops.attn_fwd(q, k, k, out=out, lse=lse, noalloc=True, balance=False)
    ref, ref_lse = ops.attn_fwd(q, k, k, balance=False)
    assert torch.equal(out, ref) and torch.equal(lse, ref_lse)
    out.fill_(7.0)
    # a plain launch (no shared last round) needs no scratch and is accepted at any size
    small_k = k[:, :, :64]
    ops.attn_fwd(q, small_k, small_k, out=out, lse=lse, noalloc=True)
    ref, _ = ops.attn_fwd(q, small_k, small_k)
    assert torch.equal(out, ref)


def test_noalloc_call_under_graph_capture(gpu):
    """The entry point is meant for code under HIP graph capture: once a first call on the device has
    been made outside capture (it looks up the scratch array's address and sets a kernel attribute),
    a captured call allocates nothing, and its replays, with eager work of the same entry point in
    between, give the eager result bit for bit every time."""
    g = torch.Generator(device=gpu).manual_seed(8)
    q, k, v = (torch.randn(1, 3, 4608, 128, generator=g, device=gpu).bfloat16() for _ in range(3))
    q2, k2, v2 = (torch.randn(1, 24, 4608, 128, generator=g, device=gpu).bfloat16() for _ in range(3))
    assert ops.launch_plan(q, k)["ranges"] > 0
    out = torch.empty_like(q)
    lse = torch.empty(1, 3, 4608, device=gpu)
    want_o, want_l = ops.attn_fwd(q, k, v)
    ops.attn_fwd(q, k, v, out=out, lse=lse, noalloc=True)   # first call on the device: outside capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.attn_fwd(q, k, v, out=out, lse=lse, noalloc=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.attn_fwd(q, k, v, out=out, lse=lse, noalloc=True)
    o2, l2 = torch.empty_like(q2), torch.empty(1, 24, 4608, device=gpu)
    for replay in range(3):
        out.zero_(); lse.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_o) and torch.equal(lse, want_l), replay
        ops.attn_fwd(q2, k2, v2, out=o2, lse=l2, noalloc=True)   # eager work on the same scratch between replays
        torch.cuda.synchronize()
