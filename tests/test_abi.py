"""The C-ABI library loads, exports every symbol include/xdit_amd_attn.h declares, its ctypes
mirror has the header's struct sizes, and argument errors come back as codes + messages
(no compute call is made: every check below fails validation before any launch)."""
import ctypes
import os
import re
import subprocess

import pytest

from xdit_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "xdit_amd_attn.h")


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(xdit_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS)
    L = _lib.lib()
    for n in names:
        assert getattr(L, n) is not None
    assert L.xdit_attn_abi_version() == _lib.ABI_VERSION


def test_ctypes_structs_match_header(tmp_path):
    c = tmp_path / "sz.c"
    c.write_text('#include "xdit_amd_attn.h"\n#include <stdio.h>\n#include <stddef.h>\n'
                 'int main(){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(xdit_attn_args), sizeof(xdit_merge_args),'
                 ' sizeof(xdit_quant_args), offsetof(xdit_attn_args, q_stride), offsetof(xdit_attn_args, stream),'
                 ' offsetof(xdit_merge_args, acc_lse_stride), sizeof(xdit_prologue_args),'
                 ' offsetof(xdit_prologue_args, x_stride), offsetof(xdit_quant_args, hadamard_block));}\n')
    exe = tmp_path / "sz"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(c), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert got == [ctypes.sizeof(_lib.AttnArgs), ctypes.sizeof(_lib.MergeArgs), ctypes.sizeof(_lib.QuantArgs),
                   _lib.AttnArgs.q_stride.offset, _lib.AttnArgs.stream.offset, _lib.MergeArgs.acc_lse_stride.offset,
                   ctypes.sizeof(_lib.PrologueArgs), _lib.PrologueArgs.x_stride.offset, _lib.QuantArgs.hadamard_block.offset]


def _attn_args(**kw):
    a = _lib.AttnArgs()
    a.struct_size = ctypes.sizeof(_lib.AttnArgs)
    a.dtype = a.out_dtype = _lib.DTYPE_BF16
    a.B, a.H, a.D = 1, 2, 128
    a.Sq = a.Sk = 64
    a.softmax_scale = 0.1
    fake = 0x1000  # never dereferenced: validation fails first
    a.q = a.k = a.v = a.out = fake
    for s in ("q_stride", "k_stride", "v_stride", "out_stride"):
        setattr(a, s, _lib.Strides(2 * 64 * 128, 64 * 128, 128))
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,code,needle", [
    (dict(struct_size=8), _lib.XDIT_ERR_INVALID_ARG, "struct_size"),
    (dict(dtype=9), _lib.XDIT_ERR_INVALID_ARG, "dtype"),
    (dict(causal=1), _lib.XDIT_ERR_UNSUPPORTED, "causal"),
    (dict(q=0), _lib.XDIT_ERR_INVALID_ARG, "q is NULL"),
    (dict(k=0x1004), _lib.XDIT_ERR_INVALID_ARG, "16-byte aligned"),
    (dict(Sk=0), _lib.XDIT_ERR_INVALID_ARG, "Sk"),
    (dict(D=100), _lib.XDIT_ERR_UNSUPPORTED, "head_dim"),
    (dict(D=512), _lib.XDIT_ERR_UNSUPPORTED, "head_dim"),
    (dict(softmax_scale=0.0), _lib.XDIT_ERR_INVALID_ARG, "softmax_scale"),
    (dict(softmax_scale=float("nan")), _lib.XDIT_ERR_INVALID_ARG, "softmax_scale"),
    (dict(out_dtype=_lib.DTYPE_FP32), _lib.XDIT_ERR_INVALID_ARG, "out_dtype"),
    (dict(v_stride=_lib.Strides(0, 0, 4)), _lib.XDIT_ERR_INVALID_ARG, "stride"),
    # tile loads form "row * stride" with a 24-bit multiply: S strides from 16 MiB up are refused
    (dict(k_stride=_lib.Strides(0, 128, 1 << 23)), _lib.XDIT_ERR_INVALID_ARG, "too large"),
    (dict(rows_per_workgroup=100), _lib.XDIT_ERR_INVALID_ARG, "rows_per_workgroup"),
    (dict(cu_count=-1), _lib.XDIT_ERR_INVALID_ARG, "cu_count"),
    (dict(Sk2=5), _lib.XDIT_ERR_INVALID_ARG, "k2 is NULL"),
    (dict(dtype=_lib.DTYPE_FP8_E4M3FN, out_dtype=_lib.DTYPE_BF16, D=96), _lib.XDIT_ERR_UNSUPPORTED, "fp8"),
])
def test_attn_fwd_rejects_bad_arguments(kw, code, needle):
    L = _lib.lib()
    rc = L.xdit_attn_fwd(ctypes.byref(_attn_args(**kw)))
    assert rc == code
    assert needle in _lib.last_error()
    with pytest.raises({_lib.XDIT_ERR_INVALID_ARG: ValueError, _lib.XDIT_ERR_UNSUPPORTED: NotImplementedError}[code]):
        _lib.check(rc)


def test_null_args_and_merge_quant_validation():
    L = _lib.lib()
    assert L.xdit_attn_fwd(None) == _lib.XDIT_ERR_INVALID_ARG
    assert L.xdit_lse_merge(None) == _lib.XDIT_ERR_INVALID_ARG
    assert L.xdit_fp8_quant(None) == _lib.XDIT_ERR_INVALID_ARG
    m = _lib.MergeArgs()
    m.struct_size = ctypes.sizeof(_lib.MergeArgs)
    m.block_dtype = _lib.DTYPE_FP8_E4M3FN
    assert L.xdit_lse_merge(ctypes.byref(m)) == _lib.XDIT_ERR_INVALID_ARG and "block_dtype" in _lib.last_error()
    m.block_dtype = _lib.DTYPE_BF16
    m.B, m.H, m.D, m.S = 1, 1, 12, 4
    assert L.xdit_lse_merge(ctypes.byref(m)) == _lib.XDIT_ERR_INVALID_ARG and "head_dim" in _lib.last_error()
    q = _lib.QuantArgs()
    q.struct_size = ctypes.sizeof(_lib.QuantArgs)
    q.in_dtype = _lib.DTYPE_FP8_E4M3FN
    assert L.xdit_fp8_quant(ctypes.byref(q)) == _lib.XDIT_ERR_INVALID_ARG and "in_dtype" in _lib.last_error()


def test_error_message_is_per_thread_and_cleared_on_entry():
    import threading
    L = _lib.lib()
    L.xdit_attn_fwd(None)
    seen = {}

    def other():
        seen["msg"] = _lib.last_error()
    t = threading.Thread(target=other)
    t.start(); t.join()
    assert seen["msg"] == "" and _lib.last_error() == "args is NULL"


def _quant_args(**kw):
    a = _lib.QuantArgs()
    a.struct_size = ctypes.sizeof(_lib.QuantArgs)
    a.in_dtype = _lib.DTYPE_BF16
    a.B, a.H, a.D, a.S = 1, 2, 128, 64
    a.x = a.y = a.descale = 0x1000
    a.x_stride = a.y_stride = _lib.Strides(2 * 64 * 128, 64 * 128, 128)
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,needle", [
    (dict(hadamard_block=48), "hadamard_block"),
    (dict(hadamard_block=256), "hadamard_block"),
    (dict(hadamard_block=-2), "hadamard_block"),
    (dict(D=96, hadamard_block=64), "hadamard_block"),
    (dict(D=4096), "head_dim"),
    (dict(descale=0), "descale"),
    (dict(y=0x1004), "8-byte aligned"),
])
def test_quant_rejects_bad_arguments(kw, needle):
    rc = _lib.lib().xdit_fp8_quant(ctypes.byref(_quant_args(**kw)))
    assert rc == _lib.XDIT_ERR_INVALID_ARG and needle in _lib.last_error()


def _prologue_args(**kw):
    a = _lib.PrologueArgs()
    a.struct_size = ctypes.sizeof(_lib.PrologueArgs)
    a.dtype = _lib.DTYPE_BF16
    a.norm, a.rope = _lib.NORM_HEAD, _lib.ROPE_INTERLEAVED
    a.B, a.H, a.D, a.S = 1, 2, 128, 64
    a.eps = 1e-6
    a.x = a.y = a.weight = a.cos = a.sin = 0x1000
    a.rope_stride, a.rope_row0, a.rope_rows = 128, 0, 64
    a.x_stride = a.y_stride = _lib.Strides(2 * 64 * 128, 64 * 128, 128)
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,code,needle", [
    (dict(struct_size=8), _lib.XDIT_ERR_INVALID_ARG, "struct_size"),
    (dict(dtype=_lib.DTYPE_FP8_E4M3FN), _lib.XDIT_ERR_INVALID_ARG, "dtype"),
    (dict(norm=7), _lib.XDIT_ERR_INVALID_ARG, "norm mode"),
    (dict(rope=9), _lib.XDIT_ERR_INVALID_ARG, "rope mode"),
    (dict(D=100), _lib.XDIT_ERR_UNSUPPORTED, "head_dim"),
    (dict(D=1024), _lib.XDIT_ERR_UNSUPPORTED, "head_dim"),
    (dict(eps=float("nan")), _lib.XDIT_ERR_INVALID_ARG, "eps"),
    (dict(cos=0), _lib.XDIT_ERR_INVALID_ARG, "cos / sin are NULL"),
    (dict(rope_stride=126), _lib.XDIT_ERR_INVALID_ARG, "row stride"),
    (dict(rope_row0=10, rope_rows=60), _lib.XDIT_ERR_INVALID_ARG, "rope rows"),
    (dict(weight=0x1002), _lib.XDIT_ERR_INVALID_ARG, "weight"),
    (dict(norm=_lib.NORM_TOKEN, H=80), _lib.XDIT_ERR_UNSUPPORTED, "token-wide norm supports"),
    (dict(norm=_lib.NORM_TOKEN, D=72, x_stride=_lib.Strides(2 * 64 * 72, 64 * 72, 72), y_stride=_lib.Strides(2 * 64 * 72, 64 * 72, 72)),
     _lib.XDIT_ERR_UNSUPPORTED, "token-wide norm needs"),
    (dict(rope=_lib.ROPE_SPLIT_HALF, D=72, rope_stride=72, x_stride=_lib.Strides(2 * 64 * 72, 64 * 72, 72),
          y_stride=_lib.Strides(2 * 64 * 72, 64 * 72, 72)), _lib.XDIT_ERR_UNSUPPORTED, "split-half"),
    (dict(y=0), _lib.XDIT_ERR_INVALID_ARG, "y is NULL"),
])
def test_prologue_rejects_bad_arguments(kw, code, needle):
    L = _lib.lib()
    assert L.xdit_qk_prologue(None) == _lib.XDIT_ERR_INVALID_ARG
    rc = L.xdit_qk_prologue(ctypes.byref(_prologue_args(**kw)))
    assert rc == code and needle in _lib.last_error()


def test_workspace_query_needs_no_gpu():
    """Sizing the balanced-launch workspace is host arithmetic: Flux-1024 at 384 query rows shares
    the last 32 of its 288 query tiles between 256 workgroups."""
    a = _attn_args(B=1, H=24, Sq=4608, Sk=4608)
    for s in ("q_stride", "k_stride", "v_stride", "out_stride"):
        setattr(a, s, _lib.Strides(24 * 4608 * 128, 4608 * 128, 128))
    need = _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(a))
    # fixed ranges of 9 KV iterations: up to 72 / 9 + 1 parts per tile; 16 KiB of counters lead every workspace
    assert need == 16384 + 32 * (72 // 9 + 1) * 384 * (128 * 2 + 4)
    a.streamed_sharing = 1   # 8 workgroups per shared tile, one partial result each
    assert _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(a)) == 16384 + 32 * 8 * 384 * (128 * 2 + 4)
    a.Sk = 64   # a single KV tile cannot be shared
    assert _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(a)) == 0


def test_workspace_of_claimed_ranges():
    """A long share (128 remaining query tiles of 256 KV iterations over 256 workgroups = 128
    iterations each) is cut into ranges of 64 iterations that workgroups claim one after the
    other: 4 (+1) slots per remaining tile, behind the 16 KiB of counters that lead a workspace."""
    a = _attn_args(B=1, H=12, Sq=32 * 384, Sk=256 * 64, rows_per_workgroup=384)
    a.q_stride = a.out_stride = _lib.Strides(12 * 32 * 384 * 128, 32 * 384 * 128, 128)
    a.k_stride = a.v_stride = _lib.Strides(12 * 256 * 64 * 128, 256 * 64 * 128, 128)
    need = _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(a))
    parts = 128 * (256 // 64 + 1) * 384 * (128 * 2 + 4)
    assert need == 16384 + parts


def test_fused_ring_step_rejects_bad_arguments():
    """xdit_attn_fwd_accumulate validates before it launches: no GPU needed for the error paths."""
    L = _lib.lib()
    a = _attn_args()
    assert L.xdit_attn_fwd_accumulate(ctypes.byref(a), None) == _lib.XDIT_ERR_INVALID_ARG and "acc is NULL" in _lib.last_error()
    r = _lib.RingAcc()
    r.struct_size = 8
    assert L.xdit_attn_fwd_accumulate(ctypes.byref(a), ctypes.byref(r)) == _lib.XDIT_ERR_INVALID_ARG and "acc struct_size" in _lib.last_error()
    r.struct_size = ctypes.sizeof(_lib.RingAcc)
    assert ctypes.sizeof(_lib.RingAcc) == 16 + 16 + 2 * 24
    r.acc_out, r.acc_lse = 0x2000, 0x3000
    r.acc_out_stride = _lib.Strides(a.H * a.Sq * a.D, a.Sq * a.D, a.D)
    r.acc_lse_stride = _lib.Strides(a.H * a.Sq, a.Sq, 1)
    f8 = _attn_args(dtype=_lib.DTYPE_FP8_E4M3FN, out_dtype=_lib.DTYPE_BF16, D=32)  # the fp8 ring step needs head_dim 128 or 64
    assert L.xdit_attn_fwd_accumulate(ctypes.byref(f8), ctypes.byref(r)) == _lib.XDIT_ERR_UNSUPPORTED and "fused ring step" in _lib.last_error()
    r.acc_out = 0x2004
    assert L.xdit_attn_fwd_accumulate(ctypes.byref(a), ctypes.byref(r)) == _lib.XDIT_ERR_INVALID_ARG and "acc_out" in _lib.last_error()
    r.acc_out = 0x2000
    r.acc_lse = 0
    assert L.xdit_attn_fwd_accumulate(ctypes.byref(a), ctypes.byref(r)) == _lib.XDIT_ERR_INVALID_ARG and "acc_lse is NULL" in _lib.last_error()
    r.acc_lse = 0x3000
    r.discard_acc_out = 1
    a.out = 0
    assert L.xdit_attn_fwd_accumulate(ctypes.byref(a), ctypes.byref(r)) == _lib.XDIT_ERR_INVALID_ARG and "discard_acc_out" in _lib.last_error()


def _plan(B, H, Sq, Sk, Sk2=0, dtype=None, D=128, rows=0, cus=0, det=True, ring_step=False, balance=0):
    a = _attn_args(B=B, H=H, Sq=Sq, Sk=Sk, Sk2=Sk2, D=D, rows_per_workgroup=rows, cu_count=cus, streamed_sharing=0 if det else 1, balance=balance)
    if dtype is not None:
        a.dtype = dtype
        a.out_dtype = _lib.DTYPE_BF16
    if Sk2:
        a.k2 = a.v2 = 0x1000
    p = _lib.LaunchPlan()
    p.struct_size = ctypes.sizeof(_lib.LaunchPlan)
    p.ring_step = 1 if ring_step else 0
    rc = _lib.lib().xdit_attn_launch_plan(ctypes.byref(a), ctypes.byref(p))
    assert rc == 0, _lib.last_error()
    if not ring_step:
        assert p.workspace_bytes == _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(a))
    return p


def test_launch_plan_invariants():
    """The launch geometry for a few hundred random problems: the ranges partition the KV iterations
    of the shared query tiles exactly, every part of a tile has a workspace slot of its own below
    slots_per_tile, the claimers fit the grid, and the workspace holds all slots (host arithmetic
    only; 256 compute units are assumed without a GPU)."""
    import random
    rng = random.Random(1234)
    seen_counter = seen_fused = seen_separate = seen_plain = 0
    for trial in range(400):
        rows_env = rng.choice([None, "128", "256", "384"])
        fp8 = rng.random() < 0.25
        B, H = rng.choice([1, 1, 2]), rng.choice([1, 3, 5, 12, 24, 40, 64])
        Sq = rng.choice([rng.randint(1, 4000), rng.randint(4000, 40000), rng.randint(40000, 130000)])
        Sk = rng.choice([rng.randint(1, 600), rng.randint(600, 20000), rng.randint(20000, 130000)])
        Sk2 = rng.choice([0, 0, rng.randint(1, 600)])
        p = _plan(B, H, Sq, Sk, Sk2, dtype=_lib.DTYPE_FP8_E4M3FN if fp8 else None, rows=int(rows_env or 0))
        rows, nt = p.rows_per_workgroup, p.kv_iterations
        assert rows in (128, 256, 384) and (rows_env is None or rows == int(rows_env))
        assert p.query_tiles == B * H * -(-Sq // rows) and nt == -(-Sk // 64) + -(-Sk2 // 64)
        if p.ranges == 0:
            seen_plain += 1
            assert p.workspace_bytes == 0 and p.whole_tiles == p.query_tiles and p.claimers == 0 and p.counter == 0
            assert p.workgroups >= p.query_tiles and p.workgroups % 8 == 0
            continue
        rem = p.query_tiles - p.whole_tiles
        work = rem * nt
        assert 0 < rem and p.range_len >= 1
        assert (p.ranges - 1) * p.range_len < work <= p.ranges * p.range_len          # exact partition
        assert 1 <= p.claimers <= p.ranges and (p.counter == 1) == (p.ranges > p.claimers)
        assert not fp8 or p.counter == 0
        if p.first_claimer + p.claimers <= p.whole_tiles:                              # claimers are whole-tile workgroups
            seen_fused += 1
            assert p.workgroups == p.whole_tiles and p.first_claimer == p.whole_tiles - p.claimers
        else:
            seen_separate += 1
            assert p.first_claimer == p.whole_tiles and p.workgroups == p.whole_tiles + p.claimers
        seen_counter += p.counter
        # slots: the parts of shared tile r are the ranges that intersect [r nt, (r+1) nt)
        for r in {0, rem - 1, rng.randrange(rem)}:
            first = (r * nt) // p.range_len
            last = ((r + 1) * nt - 1) // p.range_len
            assert last < p.ranges and last - first + 1 <= p.slots_per_tile
        parts = rem * p.slots_per_tile * rows * (128 * 2 + 4)
        assert p.workspace_bytes == 16384 + parts
    assert seen_counter > 10 and seen_fused > 10 and seen_plain > 10


def test_launch_plan_of_the_named_shapes():
    flux = _plan(1, 24, 4608, 4608)
    assert (flux.rows_per_workgroup, flux.query_tiles, flux.whole_tiles, flux.ranges, flux.range_len,
            flux.claimers, flux.first_claimer, flux.counter, flux.workgroups) == (384, 288, 256, 256, 9, 256, 0, 0, 256)
    fs = _plan(1, 24, 4608, 4608, det=False)   # the default: streamed sharing, 8 members per shared tile owning 2 iterations each
    assert (fs.rows_per_workgroup, fs.whole_tiles, fs.ranges, fs.range_len, fs.claimers, fs.first_claimer, fs.counter, fs.workgroups,
            fs.streamed, fs.slots_per_tile) == (384, 256, 256, 2, 256, 0, 1, 256, 1, 8)
    assert _plan(1, 3, 118800 + 256, 118800 + 256, det=False).streamed == 0   # long shares keep their claimed ranges
    hv = _plan(1, 3, 118800 + 256, 118800 + 256)
    assert (hv.rows_per_workgroup, hv.query_tiles, hv.whole_tiles, hv.kv_iterations) == (384, 933, 768, 1861)
    assert (hv.ranges, hv.range_len, hv.claimers, hv.first_claimer, hv.counter, hv.workgroups) == (1536, 200, 256, 512, 1, 768)
    wan = _plan(1, 5, 75600, 75600, dtype=_lib.DTYPE_FP8_E4M3FN)
    assert (wan.rows_per_workgroup, wan.whole_tiles, wan.ranges, wan.claimers, wan.counter) == (384, 768, 256, 256, 0)
    ring_chunk = _plan(1, 24, 4608, 1152)
    assert (ring_chunk.rows_per_workgroup, ring_chunk.ranges, ring_chunk.workgroups) == (256, 0, 432)   # 18 KV tiles, never balanced (the ring step folds in its epilogue)
    # tensors of a smaller head_dim run on the kernel built for the next one up, same geometry
    fields = [n for n, _ in _lib.LaunchPlan._fields_]
    for small, built in ((72, 128), (120, 128), (8, 64), (40, 64)):
        for shape in ((2, 16, 4096, 4096), (1, 5, 20000, 20000, 77)):
            a_, b_ = _plan(*shape, D=small), _plan(*shape, D=built)
            assert [getattr(a_, n) for n in fields] == [getattr(b_, n) for n in fields], (small, shape)
    # a problem too large for one launch is refused by the planning calls as by the launch
    big = _attn_args(B=40000, H=40000, Sq=64)
    p = _lib.LaunchPlan()
    p.struct_size = ctypes.sizeof(_lib.LaunchPlan)
    assert _lib.lib().xdit_attn_launch_plan(ctypes.byref(big), ctypes.byref(p)) == _lib.XDIT_ERR_INVALID_ARG
    assert _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(big)) == _lib.XDIT_ERR_INVALID_ARG
    p = _lib.LaunchPlan()
    p.struct_size = 4
    a = _attn_args()
    assert _lib.lib().xdit_attn_launch_plan(ctypes.byref(a), ctypes.byref(p)) == _lib.XDIT_ERR_INVALID_ARG
    p.struct_size = ctypes.sizeof(_lib.LaunchPlan)
    a.dtype = a.out_dtype = _lib.DTYPE_FP32
    a.D = 136   # no kernel takes fp32 tensors of a head_dim above 128
    assert _lib.lib().xdit_attn_launch_plan(ctypes.byref(a), ctypes.byref(p)) == _lib.XDIT_ERR_UNSUPPORTED


def test_launch_choice_against_measured_option_times():
    """The library's choice of launch (query rows per workgroup, balanced or not) held to
    measurements: tests/golden/launch_option_times.json records the settled time of every launch
    option for 180-odd problems on a 256-compute-unit MI355X (16-bit at head_dim 64..128 and fp8;
    self-attention, ring chunks, cross-attention, long sequences, random shapes).  For every
    problem the option `xdit_attn_launch_plan` picks (planned for 256 compute units) must be
    within 15 % of the fastest recorded option, and within 3 % on average per dtype."""
    import json
    data = json.load(open(os.path.join(ROOT, "tests", "golden", "launch_option_times.json")))
    assert len(data["problems"]) > 150
    loss = {"bf16": [], "fp8": []}
    for pr in data["problems"]:
        B, H, Sq, Sk, D = pr["shape"]
        p = _plan(B, H, Sq, Sk, dtype=_lib.DTYPE_FP8_E4M3FN if pr["dtype"] == "fp8" else None, D=D, cus=data["cu_count"])
        times = {(rows, bal): t for rows, bal, t in pr["options"]}
        chosen = (p.rows_per_workgroup, 2 if p.ranges else 1)
        assert chosen in times, (pr["shape"], chosen)
        excess = times[chosen] / min(times.values()) - 1.0
        assert excess <= 0.15, (pr["dtype"], pr["shape"], chosen, times)
        loss[pr["dtype"]].append(excess)
    for dtype, xs in loss.items():
        assert len(xs) > 40 and sum(xs) / len(xs) <= 0.03, (dtype, sum(xs) / len(xs))


WALK_HARNESS = r"""
// Walks every workgroup of a planned launch with the code the kernels run (attn_walk.h) and
// checks the coverage: stdin holds one launch per line.
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "attn_walk.h"
struct Geom { int total_tiles, tiles_per_xcd, split_full, split_units, split_len, split_pmax, split_fuse0, split_claimers, split_dyn, split_s0, split_order; };
int main() {
  Geom g; int nt, workgroups, counter, order; long line = 0;
  int fold;
  while (scanf("%d %d %d %d %d %d %d %d %d %d %d %d %d %d %d %d", &g.total_tiles, &g.tiles_per_xcd, &g.split_full, &g.split_units, &g.split_len,
               &g.split_pmax, &g.split_fuse0, &g.split_claimers, &nt, &workgroups, &counter, &order, &g.split_dyn, &g.split_s0, &g.split_order, &fold) == 16) {
    line++;
    // fold duties (launches that fold inside the kernel): the word of every shared tile, which rows have been folded, and
    // per workgroup the duties it has put off to its end (parts-first launches)
    const int ROWS = 384;
    std::vector<unsigned> word(g.total_tiles, 0u);
    std::vector<int> folded((size_t)(fold ? (g.total_tiles - g.split_full) * ROWS : 0), 0);
    std::vector<int> arrived(g.total_tiles, 0);
    std::vector<std::vector<int>> duties(workgroups);
    auto fold_now = [&](int r, unsigned mask, int n) {
      if (mask && arrived[r] != n) { printf("line %ld: tile %d folded before its parts were there\n", line, r); exit(1); }
      for (int j = 0; j < n; j++) if ((mask >> j) & 1u) { int r0, r1; xdit::fold_slice_rows(j, n, ROWS, r0, r1); for (int x = r0; x < r1; x++) folded[(size_t)r * ROWS + x]++; }
    };
    auto event = [&](int r, int j, int n, bool arrival, bool with_duty) {
      const unsigned add = arrival ? xdit::fold_arrive_word(j, with_duty) : xdit::fold_duty_word(j);
      const unsigned old = word[r];
      word[r] += add;
      if (arrival) arrived[r]++;
      fold_now(r, arrival ? xdit::fold_after_arrival(old, j, with_duty, n) : xdit::fold_after_duty(old, j, n), n);
      if (xdit::fold_last_event(old, add, n)) word[r] = 0u;
    };
    std::vector<unsigned> tile_counter(g.total_tiles, 0u);
    std::vector<int> cover((size_t)g.total_tiles * nt, 0);
    const int rem = g.total_tiles - g.split_full;
    std::vector<int> slot_used((size_t)(g.split_units ? rem * g.split_pmax : 0), 0);
    std::vector<xdit::WorkgroupWalk> walk(workgroups);
    std::vector<char> live(workgroups, 0);
    unsigned ticket = 0;
    for (int w = 0; w < workgroups; w++) live[w] = walk[w].start(g, nt, w);
    // order 0: a workgroup runs to its end before the next starts; 1: the reverse; 2: one segment per workgroup in turn
    bool any = true;
    auto step = [&](int w) {
      xdit::Segment s;
      if (!walk[w].next(g, nt, s)) {
        live[w] = 0;
        for (size_t d = 0; d + 2 < duties[w].size(); d += 3) event(duties[w][d], duties[w][d + 1], duties[w][d + 2], false, false);  // at the workgroup's end
        if (g.split_order != 0) {  // the kernel works the duties out again from the workgroup's index: the same ones
          std::vector<int> again;
          const int u = w - g.split_fuse0, rem_iters = (g.total_tiles - g.split_full) * nt;
          if (u >= 0 && u < g.split_units)
            for (int lin = u * g.split_len, lin_end = lin + g.split_len < rem_iters ? lin + g.split_len : rem_iters; lin < lin_end;) {
              const int r = lin / nt, it1 = lin_end - r * nt < nt ? lin_end - r * nt : nt;
              again.push_back(r); again.push_back(u - (r * nt) / g.split_len); again.push_back(xdit::shared_tile_parts(g, nt, r));
              lin = r * nt + it1;
            }
          if (again != duties[w]) { printf("line %ld: duties of workgroup %d\n", line, w); exit(1); }
        }
        return;
      }
      if (s.tile < 0 || s.tile >= g.total_tiles || s.it0 < 0 || s.it1 > nt || s.it0 >= s.it1) { printf("line %ld: bad segment\n", line); exit(1); }
      for (int t = s.it0; t < s.it1; t++) cover[(size_t)s.tile * nt + t]++;
      if (s.dyn >= 0) {  // streamed sharing: draw the tile's other iterations one at a time, as the kernel does
        if (s.tile != g.split_full + s.dyn || s.pool0 < s.it1 || !g.split_dyn) { printf("line %ld: bad streamed segment\n", line); exit(1); }
        // order 2 interleaves the draws of the group's members; the others let one member take the whole pool
        for (int n = 0; order != 2 || n < 3; n++) {
          const unsigned tk = tile_counter[s.dyn]++;
          if ((int)tk >= nt - s.pool0) break;
          cover[(size_t)s.tile * nt + s.pool0 + tk]++;
        }
      }
      if (s.slot >= 0) {
        if (s.tile < g.split_full || s.slot >= (long)slot_used.size()) { printf("line %ld: bad slot\n", line); exit(1); }
        const int r = s.tile - g.split_full;
        if (s.slot / g.split_pmax != r || s.slot % g.split_pmax >= xdit::shared_tile_parts(g, nt, r)) { printf("line %ld: slot outside its tile\n", line); exit(1); }
        slot_used[s.slot]++;
        if (fold) {
          const int n = xdit::shared_tile_parts(g, nt, r), j = (int)(s.slot % g.split_pmax);
          if (n > xdit::kFoldMaxParts) { printf("line %ld: %d parts in a launch that folds in the kernel\n", line, n); exit(1); }
          event(r, j, n, true, g.split_order == 0);
          if (g.split_order != 0) { duties[w].push_back(r); duties[w].push_back(j); duties[w].push_back(n); }
        }
      } else if (s.it0 != 0 || s.it1 != nt) { printf("line %ld: partial tile without a slot\n", line); exit(1); }
      if (walk[w].wants_claim(counter != 0 && !g.split_dyn)) walk[w].claimed(g, ticket++);
    };
    while (any) {
      any = false;
      for (int i = 0; i < workgroups; i++) {
        const int w = order == 1 ? workgroups - 1 - i : i;
        if (order == 2) { if (live[w]) { step(w); any = true; } }
        else while (live[w]) step(w);
      }
    }
    if (g.split_dyn)  // whoever comes last drains what is left of every pool (the kernel's members draw until the pool is empty)
      for (int r = 0; r < rem; r++) {
        const int pool0 = xdit::shared_tile_parts(g, nt, r) * g.split_s0;
        for (;;) { const unsigned tk = tile_counter[r]++; if ((int)tk >= nt - pool0) break; cover[(size_t)(g.split_full + r) * nt + pool0 + tk]++; }
      }
    for (size_t i = 0; i < cover.size(); i++)
      if (cover[i] != 1) { printf("line %ld: tile %zu iteration %zu covered %d times\n", line, i / nt, i % nt, cover[i]); return 1; }
    for (size_t i = 0; i < folded.size(); i++)
      if (folded[i] != 1) { printf("line %ld: row %zu of shared tile %zu folded %d times\n", line, i % ROWS, i / ROWS, folded[i]); return 1; }
    for (int r = 0; r < (fold ? rem : 0); r++)
      if (word[r] != 0u) { printf("line %ld: fold word of tile %d left at %u\n", line, r, word[r]); return 1; }
    for (int r = 0; r < (g.split_units ? rem : 0); r++)
      for (int k = 0; k < g.split_pmax; k++)
        if (slot_used[(size_t)r * g.split_pmax + k] != (k < xdit::shared_tile_parts(g, nt, r) ? 1 : 0)) { printf("line %ld: slots of tile %d\n", line, r); return 1; }
  }
  printf("ok %ld\n", line);
  // thread -> row map of the merge kernel: every chunk of every row held exactly once, by lanes of one wavefront
  for (int cpr = 1; cpr <= 64; cpr++) {
    const xdit::MergeMap m = xdit::merge_map(cpr * 8);
    const int rows = 1000;
    std::vector<int> held((size_t)rows * cpr, 0);
    std::vector<long> wave_of(rows, -1);
    const long waves = (rows + m.rows_per_wave - 1) / m.rows_per_wave;
    for (long wv = 0; wv < waves; wv++)
      for (int lane = 0; lane < 64; lane++) {
        int64_t row; int c0;
        if (lane / m.lanes_per_row != (int)((lane * m.inv) >> 16)) { printf("merge map: division cpr %d\n", cpr); return 1; }
        if (!xdit::merge_thread_row(m, wv, lane, row, c0) || row >= rows) continue;
        if (wave_of[row] >= 0 && wave_of[row] != wv) { printf("merge map: row %ld in two wavefronts, cpr %d\n", (long)row, cpr); return 1; }
        wave_of[row] = wv;
        held[(size_t)row * cpr + c0]++;
      }
    for (size_t i = 0; i < held.size(); i++) if (held[i] != 1) { printf("merge map: cpr %d chunk held %d times\n", cpr, held[i]); return 1; }
  }
  printf("merge map ok\n");
  return 0;
}
"""


def test_every_tile_and_kv_iteration_is_covered_exactly_once(tmp_path):
    """Coverage of planned launches, walked on the CPU with the very code the kernels run
    (csrc/attn_walk.h compiled by g++): for compute-unit counts 1..304 (multiples of 8 or not) and
    random problems, every (query tile, KV iteration) is processed exactly once, every part of a
    shared tile lands in a slot of its own among those the fold reads, under three execution
    orders of the workgroups; and where the kernel folds the shared tiles itself, the fold-duty
    protocol folds every row of every shared tile exactly once, never before all of the tile's
    parts are there, and leaves the tiles' words at zero.  Also the merge kernel's thread -> row map for head_dim 8..512."""
    import random
    src = tmp_path / "walk.cpp"
    src.write_text(WALK_HARNESS)
    exe = tmp_path / "walk"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-I", os.path.join(ROOT, "xdit_amd", "csrc"), str(src), "-o", str(exe)])
    rng = random.Random(99)
    lines, balanced, odd_balanced, streamed, folds, parts_first = [], 0, 0, 0, 0, 0
    cases = [(cus, None) for cus in range(1, 305)] + [(rng.choice([0, 8, 64, 100, 252, 255, 256, 304]), i) for i in range(300)]
    for cus, extra in cases:
        fp8 = rng.random() < 0.25
        rows = rng.choice([0, 128, 256, 384])
        B, H = rng.choice([1, 2]), rng.choice([1, 3, 5, 12, 24])
        Sq = rng.choice([rng.randint(1, 3000), rng.randint(3000, 40000), rng.randint(3000, 40000)])
        Sk = rng.choice([rng.randint(1, 600), rng.randint(3500, 12000), rng.randint(3500, 12000)])
        Sk2 = rng.choice([0, 0, rng.randint(1, 300)])
        ring_step = rng.random() < 0.5
        p = _plan(B, H, Sq, Sk, Sk2, dtype=_lib.DTYPE_FP8_E4M3FN if fp8 else None, rows=rows, cus=cus, det=rng.random() < 0.3,
                  ring_step=ring_step, balance=2 if ring_step else 0)
        assert p.fold_in_kernel == (1 if ring_step and p.ranges else 0) and (ring_step or not p.parts_first)
        streamed += p.streamed
        fuse0 = p.first_claimer if p.ranges and p.first_claimer + p.claimers <= p.whole_tiles else 0x7fffffff
        full = p.whole_tiles if p.ranges else 0
        balanced += p.ranges > 0
        odd_balanced += p.ranges > 0 and full % 8 != 0
        for order in (0, 1, 2):
            lines.append("%d %d %d %d %d %d %d %d %d %d %d %d %d %d %d %d" % (p.query_tiles, -(-p.query_tiles // 8), full, p.ranges, p.range_len,
                                                                         p.slots_per_tile, fuse0, p.claimers, p.kv_iterations, p.workgroups, p.counter, order,
                                                                         p.streamed, p.range_len if p.streamed else 0, p.parts_first, p.fold_in_kernel))
        folds += p.fold_in_kernel
        parts_first += p.parts_first
    assert balanced > 100 and odd_balanced > 20 and streamed > 20 and folds > 50 and parts_first > 10 and balanced - folds > 50
    out = subprocess.run([str(exe)], input="\n".join(lines) + "\n", capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.split("\n")[0] == "ok %d" % len(lines) and "merge map ok" in out.stdout, out.stdout[-400:]


def test_launch_plan_of_the_fp32_kernel():
    """fp32 problems run one workgroup per query tile: 128-row tiles with 32-key KV tiles, or
    64-row tiles with 64-key KV tiles when the 128-row tiles would fill less than three quarters
    of the compute units the launch is planned for."""
    p = _plan(1, 16, 1024, 1024, dtype=_lib.DTYPE_FP32, D=72, cus=256)      # PixArt-512: 128 tiles of 128 rows
    assert (p.rows_per_workgroup, p.query_tiles, p.kv_iterations, p.workgroups, p.workspace_bytes, p.ranges) == (64, 256, 16, 256, 0, 0)
    p = _plan(2, 16, 4096, 4096, dtype=_lib.DTYPE_FP32, D=72, cus=256)      # PixArt-1024: 1024 tiles
    assert (p.rows_per_workgroup, p.query_tiles, p.kv_iterations, p.whole_tiles) == (128, 1024, 128, 1024)
    p = _plan(1, 3, 8192, 100, Sk2=40, dtype=_lib.DTYPE_FP32, D=128, cus=256)  # 192 tiles: exactly three quarters
    assert (p.rows_per_workgroup, p.kv_iterations) == (128, 4 + 2)
    p = _plan(1, 3, 8192, 100, Sk2=40, dtype=_lib.DTYPE_FP32, D=128, cus=304)
    assert (p.rows_per_workgroup, p.query_tiles, p.kv_iterations, p.workgroups) == (64, 384, 2 + 1, 384)
    p = _plan(1, 1, 70, 10, dtype=_lib.DTYPE_FP32, D=8, cus=1)              # planned for one compute unit
    assert (p.rows_per_workgroup, p.query_tiles, p.workgroups) == (128, 1, 8)
