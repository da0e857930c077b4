"""Tensor-level entry points: torch tensors in, C ABI calls out.

Tensors are logical (B, H, S, D) with arbitrary B/H/S strides and a unit D stride, so both
BHSD-contiguous tensors and BSHD-contiguous tensors viewed as BHSD are consumed without a copy.
PyTorch is used for device memory and the current stream only.
"""
import ctypes
import threading

import torch

from . import _lib

_DTYPE_CODE = {
    torch.bfloat16: _lib.DTYPE_BF16,
    torch.float16: _lib.DTYPE_FP16,
    torch.float32: _lib.DTYPE_FP32,
    torch.float8_e4m3fn: _lib.DTYPE_FP8_E4M3FN,
}


def _code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError("unsupported dtype %s" % (dtype,))


def _strides(t):
    return _lib.Strides(t.stride(0), t.stride(1), t.stride(2))


def _check4(name, t, device):
    if not isinstance(t, torch.Tensor) or t.ndim != 4:
        raise ValueError("%s must be a 4-D tensor (B, H, S, D)" % name)
    if t.device != device:
        raise ValueError("%s is on %s, expected %s" % (name, t.device, device))
    if not t.is_cuda:
        raise RuntimeError("%s is not on a GPU: the attention kernels are HIP-only, there is no CPU path" % name)
    if t.shape[-1] > 1 and t.stride(-1) != 1:
        raise ValueError("%s must have a unit stride over head_dim" % name)


def _stream(device):
    return torch._C._cuda_getCurrentRawStream(device.index if device.index is not None else torch.cuda.current_device())


class _on_device:
    """`with torch.cuda.device(device)` only when the device is not the current one already."""
    __slots__ = ("ctx",)

    def __init__(self, device):
        idx = device.index
        self.ctx = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


_WORKSPACE = {}
_RETIRED = []


def _workspace(device, stream, nbytes):
    """Per-device scratch tensor for balanced launches, grown on demand -> [tensor, preserved].
    Calls on one stream are ordered, so one buffer per (device, stream) is reused from call to
    call; nothing else ever writes it, which is what `workspace_preserved` tells the library once
    a call on the buffer has returned without error (the caller sets entry[1] then).  A buffer that has become too small is kept alive rather than freed, so
    that its address cannot come back as a new buffer with foreign contents."""
    key = (device, stream)
    entry = _WORKSPACE.get(key)
    if entry is None or entry[0].numel() < nbytes:
        if entry is not None:
            _RETIRED.append(entry[0])
        entry = [torch.empty(int(nbytes), dtype=torch.uint8, device=device), 0]
        _WORKSPACE[key] = entry
    return entry   # [tensor, preserved]: preserved is 0 until a call on the buffer has succeeded


# Launch tuning passed to the library with every attention call (fields of xdit_attn_args):
# rows_per_workgroup 0 = the library's choice, else 128 / 256 / 384; cu_count 0 = the device's
# compute units, else plan the launch as for that many; balance 0 = the library decides whether a
# launch is balanced, 1 = never, 2 = whenever its planner offers a plan; streamed 1 = opt in to
# streamed sharing (results then reproducible to rounding only).  Tests and sweeps set these.
TUNING = {"rows_per_workgroup": 0, "cu_count": 0, "streamed": 0, "balance": 0}

# Argument structs are filled once per call signature (shapes, strides, dtypes, options) and kept:
# a later call with the same signature only patches the pointers and the stream.  One set per
# thread: the structs are patched in place, and the C call that reads them releases the GIL.
_TLS = threading.local()
_PLANS_MAX = 512


class _AttnPlan:
    __slots__ = ("args", "need", "shape", "out_dtype", "ring")


def _sig(t):
    return None if t is None else (t.shape, t.stride(), t.device, t.dtype)


def _build_attn_plan(q, k, v, softmax_scale, causal, k2, v2, descales, out_dtype, out, lse, acc, streamed):
    device = q.device
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check4(name, t, device)
    B, H, Sq, D = q.shape
    if k.shape[0] != B or k.shape[1] != H or k.shape[3] != D or v.shape != k.shape:
        raise ValueError("q %s, k %s, v %s do not agree (Hq must equal Hk)" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k, v must share a dtype")
    a = _lib.AttnArgs()
    a.struct_size = ctypes.sizeof(_lib.AttnArgs)
    a.dtype = _code(q.dtype)
    a.out_dtype = _code(out_dtype)
    a.causal = 1 if causal else 0
    a.B, a.H, a.D = B, H, D
    a.rows_per_workgroup = int(TUNING["rows_per_workgroup"])
    a.cu_count = int(TUNING["cu_count"])
    a.balance = int(TUNING["balance"])
    a.streamed_sharing = 1 if streamed else 0
    a.Sq, a.Sk = Sq, k.shape[2]
    a.softmax_scale = float(softmax_scale)
    a.q_stride, a.k_stride, a.v_stride = _strides(q), _strides(k), _strides(v)
    if k2 is not None:
        _check4("k2", k2, device)
        _check4("v2", v2, device)
        if k2.shape[0] != B or k2.shape[1] != H or k2.shape[3] != D or v2.shape != k2.shape or k2.dtype != q.dtype or v2.dtype != q.dtype:
            raise ValueError("joint k2/v2 do not match q/k/v")
        if k2.shape[2] > 0:
            a.Sk2 = k2.shape[2]
            a.k2_stride, a.v2_stride = _strides(k2), _strides(v2)
    if out is not None:
        _check4("out", out, device)
        if tuple(out.shape) != (B, H, Sq, D) or out.dtype != out_dtype:
            raise ValueError("out has the wrong shape or dtype")
        a.out_stride = _strides(out)
    else:
        a.out_stride = _lib.Strides(H * Sq * D, Sq * D, D)  # a new BHSD-contiguous tensor per call
    if lse is not None:
        if lse.dtype != torch.float32 or tuple(lse.shape) != (B, H, Sq) or lse.device != device or (Sq > 1 and lse.stride(2) != 1):
            raise ValueError("lse must be a (B, H, Sq) fp32 tensor on %s with a unit stride over Sq" % (device,))
        a.lse_stride_b, a.lse_stride_h = lse.stride(0), lse.stride(1)
    else:
        a.lse_stride_b, a.lse_stride_h = H * Sq, Sq
    for name, d in zip(("q_descale", "k_descale", "v_descale"), descales):
        if d is None:
            continue
        if q.dtype != torch.float8_e4m3fn:
            raise ValueError("%s is only meaningful for fp8 inputs" % name)
        if d.dtype != torch.float32 or tuple(d.shape) != (B, H) or d.device != device:
            raise ValueError("%s must be a (B, H) fp32 tensor on %s" % (name, device))
        a.descale_stride_b, a.descale_stride_h = H, 1  # descales are passed contiguous
    plan = _AttnPlan()
    plan.args = a
    plan.shape = (B, H, Sq, D)
    plan.out_dtype = out_dtype
    plan.ring = None
    plan.need = 0
    if acc is not None:
        acc_out, acc_lse, first, discard = acc
        _check4("acc_out", acc_out, device)
        if acc_out.dtype != torch.float32 or acc_lse.dtype != torch.float32:
            raise ValueError("acc_out and acc_lse must be fp32")
        if tuple(acc_out.shape) != (B, H, Sq, D) or tuple(acc_lse.shape) != (B, H, Sq) or acc_lse.device != device:
            raise ValueError("accumulator shape mismatch")
        r = _lib.RingAcc()
        r.struct_size = ctypes.sizeof(_lib.RingAcc)
        r.first = 1 if first else 0
        r.discard_acc_out = 1 if discard else 0
        r.acc_out_stride = _strides(acc_out)
        r.acc_lse_stride = _lib.Strides(acc_lse.stride(0), acc_lse.stride(1), acc_lse.stride(2))
        plan.ring = r
    with _on_device(device):
        if acc is None:
            need = _lib.lib().xdit_attn_workspace_bytes(ctypes.byref(a))
        else:
            # the ring step is planned on its own (its shared tiles are folded inside the kernel): its
            # launch plan says what it asks for; 0 where it has no plan (the call itself reports why)
            lp = _lib.LaunchPlan()
            lp.struct_size = ctypes.sizeof(_lib.LaunchPlan)
            lp.ring_step = 1
            need = lp.workspace_bytes if _lib.lib().xdit_attn_launch_plan(ctypes.byref(a), ctypes.byref(lp)) == 0 else 0
    if need < 0:
        _lib.check(need)
    plan.need = need
    return plan


def attn_fwd(q, k, v, softmax_scale=None, causal=False, k2=None, v2=None,
             q_descale=None, k_descale=None, v_descale=None, out_dtype=None, out=None,
             return_lse=True, balance=True, lse=None, noalloc=False, streamed=None, _acc=None):
    """Non-causal attention forward on logical BHSD tensors -> (out BHSD, lse (B,H,Sq) fp32).

    `k2`/`v2` are an optional second key/value segment (the joint text tokens) attended together
    with `k`/`v`.  For fp8 (torch.float8_e4m3fn) inputs the descales are (B, H) fp32 tensors.
    `out` / `lse` receive the results when given (new tensors otherwise).
    `balance=False` withholds the scratch buffer with which the library evens out the last round
    of workgroups (results then come from one workgroup per query tile).
    Results are reproducible bit for bit from call to call, as those of the vendor forwards behind
    the reference's adapters are; `streamed=True` opts in to a balanced launch that shares the KV
    iterations of a query tile dynamically (a per cent or two faster on some shapes, results then
    reproducible to rounding only).
    `noalloc=True` goes through the library's entry point that allocates nothing: the scratch is
    a fixed buffer inside the library (problems that need more than it holds raise ValueError
    unless `balance=False` asks for the plain launch), and `out` (and `lse` when `return_lse`)
    must be given.
    """
    if (k2 is None) != (v2 is None):
        raise ValueError("k2 and v2 should be None or not None simultaneously.")
    if not isinstance(q, torch.Tensor) or q.ndim != 4:
        raise ValueError("q must be a 4-D tensor (B, H, S, D)")
    device = q.device
    if out_dtype is None:
        out_dtype = torch.bfloat16 if q.dtype == torch.float8_e4m3fn else q.dtype
    if softmax_scale is None:
        softmax_scale = float(q.shape[-1]) ** -0.5
    if noalloc and (out is None or (return_lse and lse is None) or _acc is not None):
        raise ValueError("noalloc needs out (and lse) from the caller and is not available for the ring step")
    if lse is not None:
        return_lse = True
    if streamed is None:
        streamed = bool(TUNING["streamed"])
    acc_sig = None if _acc is None else (_sig(_acc[0]), _sig(_acc[1]), _acc[2], _acc[3])
    key = (q.dtype, out_dtype, device, _sig(q), _sig(k), _sig(v), _sig(k2), _sig(v2), _sig(out), _sig(lse),
           k.dtype, v.dtype, float(softmax_scale), bool(causal), q_descale is not None, k_descale is not None,
           v_descale is not None, acc_sig, TUNING["rows_per_workgroup"], TUNING["cu_count"], TUNING["balance"], bool(streamed))
    plans = _TLS.__dict__.setdefault("plans", {})
    plan = plans.get(key)
    if plan is None:
        plan = _build_attn_plan(q, k, v, softmax_scale, causal, k2, v2, (q_descale, k_descale, v_descale),
                                out_dtype, out, lse, _acc, streamed)
        if len(plans) >= _PLANS_MAX:
            plans.clear()
        plans[key] = plan
    else:
        for d in (q_descale, k_descale, v_descale):  # values the signature does not cover
            if d is not None and (d.dtype != torch.float32 or tuple(d.shape) != plan.shape[:2] or d.device != device):
                raise ValueError("descales must be (B, H) fp32 tensors on %s" % (device,))
    if out is None and _acc is None:
        out = torch.empty(plan.shape, dtype=out_dtype, device=device)
    if lse is None and return_lse and _acc is None:
        lse = torch.empty(plan.shape[:3], dtype=torch.float32, device=device)
    a = plan.args
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    if a.Sk2:
        a.k2, a.v2 = k2.data_ptr(), v2.data_ptr()
    a.out = out.data_ptr() if out is not None else None
    a.lse = lse.data_ptr() if lse is not None else None
    keep = None
    if q_descale is not None or k_descale is not None or v_descale is not None:
        keep = [None if d is None else d.contiguous() for d in (q_descale, k_descale, v_descale)]
        a.q_descale, a.k_descale, a.v_descale = (None if d is None else d.data_ptr() for d in keep)
    stream = _stream(device)
    a.stream = stream
    L = _lib.lib()
    entry = None
    with _on_device(device):
        if noalloc:
            a.workspace, a.workspace_bytes = None, 0
            if not balance:
                a.balance = 1   # plain launch: no scratch at all, whatever the size
            rc = L.xdit_attn_fwd_noalloc(ctypes.byref(a))
            a.balance = int(TUNING["balance"])
        else:
            if balance and plan.need > 0:
                entry = _workspace(device, stream, plan.need)
                a.workspace, a.workspace_bytes, a.workspace_preserved = entry[0].data_ptr(), entry[0].numel(), entry[1]
            else:
                a.workspace, a.workspace_bytes, a.workspace_preserved = None, 0, 0
            if _acc is not None:
                r = plan.ring
                r.acc_out, r.acc_lse = _acc[0].data_ptr(), _acc[1].data_ptr()
                rc = L.xdit_attn_fwd_accumulate(ctypes.byref(a), ctypes.byref(r))
            else:
                rc = L.xdit_attn_fwd(ctypes.byref(a))
    if entry is not None:
        entry[1] = 1 if rc == 0 else 0   # after a failure the next call has the counters cleared again
    if rc != 0:
        _lib.check(rc)
    return out, lse


def launch_plan(q, k, k2=None, streamed=None, ring_step=False):
    """How `attn_fwd(q, k, v, k2=..)` would be launched (a dict of the fields of xdit_launch_plan):
    rows per workgroup, query tiles, whole tiles, shared ranges and their length, claimers,
    whether ranges are handed out through the counter, workgroups, workspace bytes.  Host
    arithmetic only; bf16 / fp16 / fp32 (head_dim up to 128) and fp8 (head_dim 128 or 64)."""
    a = _lib.AttnArgs()
    a.struct_size = ctypes.sizeof(_lib.AttnArgs)
    a.dtype = _code(q.dtype)
    a.out_dtype = _code(torch.bfloat16 if q.dtype == torch.float8_e4m3fn else q.dtype)
    a.B, a.H, a.Sq, a.D = q.shape
    a.Sk = k.shape[2]
    a.Sk2 = 0 if k2 is None else k2.shape[2]
    a.rows_per_workgroup = int(TUNING["rows_per_workgroup"])
    a.cu_count = int(TUNING["cu_count"])
    a.balance = int(TUNING["balance"])
    a.streamed_sharing = 1 if (TUNING["streamed"] if streamed is None else streamed) else 0
    p = _lib.LaunchPlan()
    p.struct_size = ctypes.sizeof(_lib.LaunchPlan)
    p.ring_step = 1 if ring_step else 0   # the launch of attn_fwd_accumulate instead of attn_fwd's
    _lib.check(_lib.lib().xdit_attn_launch_plan(ctypes.byref(a), ctypes.byref(p)))
    return {name: getattr(p, name) for name, _ in _lib.LaunchPlan._fields_ if name != "struct_size"}


def fused_ring_step_supported(q):
    """Whether `attn_fwd_accumulate` takes these queries (bf16 / fp16 / fp32 with head_dim a multiple
    of 8 up to 128, fp8 with head_dim 128 or 64)."""
    if q.dtype == torch.float8_e4m3fn:
        return q.shape[-1] in (128, 64)
    return q.dtype in (torch.bfloat16, torch.float16, torch.float32) and q.shape[-1] % 8 == 0 and 0 < q.shape[-1] <= 128


def attn_fwd_accumulate(q, k, v, acc_out, acc_lse, first=False, final_out=None, discard_acc_out=False,
                        softmax_scale=None, k2=None, v2=None, q_descale=None, k_descale=None, v_descale=None,
                        out_dtype=None, balance=True):
    """One ring step in one launch: attention of q over (k, v) [+ (k2, v2)] folded into the fp32
    accumulator (acc_out logical BHSD, acc_lse logical BHS; any strides) exactly as `attn_fwd`
    followed by `lse_merge` would, without the block ever reaching memory.  `first` initialises
    the accumulator; `final_out` (logical BHSD, q's dtype; bf16 or fp16 for fp8 inputs) also
    receives the merged rows; `discard_acc_out` skips the write-back of acc_out (last step).
    fp8 inputs take (B, H) fp32 descales and `out_dtype` (bf16 by default), the dtype the block is
    rounded to before the fold.  Returns (acc_out, acc_lse)."""
    if discard_acc_out and final_out is None:
        raise ValueError("discard_acc_out needs final_out")
    if out_dtype is None and final_out is not None:
        out_dtype = final_out.dtype
    attn_fwd(q, k, v, softmax_scale=softmax_scale, k2=k2, v2=v2, out=final_out, return_lse=False,
             q_descale=q_descale, k_descale=k_descale, v_descale=v_descale, out_dtype=out_dtype, balance=balance,
             _acc=(acc_out, acc_lse, bool(first), bool(discard_acc_out)))
    return acc_out, acc_lse


def lse_merge(acc_out, acc_lse, block_out, block_lse, first=False, final_out=None):
    """One fold of the ring merge, in place on (acc_out fp32 BHSD-logical, acc_lse fp32 BHS-logical).

    All tensors are given as LOGICAL (B,H,S,D) / (B,H,S) views (any strides, unit D stride).
    """
    device = block_out.device
    _check4("acc_out", acc_out, device)
    _check4("block_out", block_out, device)
    if acc_out.dtype != torch.float32 or acc_lse.dtype != torch.float32 or block_lse.dtype != torch.float32:
        raise ValueError("acc_out, acc_lse and block_lse must be fp32")
    B, H, S, D = block_out.shape
    if tuple(acc_out.shape) != (B, H, S, D) or tuple(acc_lse.shape) != (B, H, S) or tuple(block_lse.shape) != (B, H, S):
        raise ValueError("shape mismatch between accumulator and block")
    a = _lib.MergeArgs()
    a.struct_size = ctypes.sizeof(_lib.MergeArgs)
    a.block_dtype = _code(block_out.dtype)
    a.first = 1 if first else 0
    a.B, a.H, a.D, a.S = B, H, D, S
    a.acc_out, a.acc_lse = acc_out.data_ptr(), acc_lse.data_ptr()
    a.block_out, a.block_lse = block_out.data_ptr(), block_lse.data_ptr()
    a.acc_out_stride, a.block_out_stride = _strides(acc_out), _strides(block_out)
    a.acc_lse_stride = _lib.Strides(acc_lse.stride(0), acc_lse.stride(1), acc_lse.stride(2))
    a.block_lse_stride = _lib.Strides(block_lse.stride(0), block_lse.stride(1), block_lse.stride(2))
    if final_out is not None:
        _check4("final_out", final_out, device)
        if tuple(final_out.shape) != (B, H, S, D):
            raise ValueError("final_out shape mismatch")
        a.final_out = final_out.data_ptr()
        a.final_dtype = _code(final_out.dtype)
        a.final_out_stride = _strides(final_out)
    a.stream = _stream(device)
    with _on_device(device):
        _lib.check(_lib.lib().xdit_lse_merge(ctypes.byref(a)))
    return acc_out, acc_lse


_QUANT_SCRATCH = {}


def fp8_quant(x, per_tensor=False, scale=None, hadamard_block=0, x2=None):
    """Abs-max fp8 quantiser on a logical BHSD tensor -> (y float8_e4m3fn BHSD-contiguous,
    descale (B,H) fp32).  `per_tensor` takes one abs-max over the whole tensor (the reference's
    per_tensor_quant); `scale` (a one-element fp32 tensor) is a static scale; `hadamard_block`
    (a power of two dividing head_dim) rotates the rows by a block Hadamard matrix first.
    `x2` (logical (B,H,S2,D), e.g. the joint keys) is quantised with the same scales, the abs-max
    taken over both tensors; the result is then (y, y2, descale)."""
    device = x.device
    _check4("x", x, device)
    B, H, S, D = x.shape
    y = torch.empty((B, H, S, D), dtype=torch.float8_e4m3fn, device=device)
    descale = torch.empty((B, H), dtype=torch.float32, device=device)
    a = _lib.QuantArgs()
    a.struct_size = ctypes.sizeof(_lib.QuantArgs)
    a.in_dtype = _code(x.dtype)
    a.per_tensor = 1 if per_tensor else 0
    a.hadamard_block = int(hadamard_block)
    a.B, a.H, a.D, a.S = B, H, D, S
    a.x, a.y, a.descale = x.data_ptr(), y.data_ptr(), descale.data_ptr()
    y2 = None
    if x2 is not None:
        _check4("x2", x2, device)
        if x2.shape[0] != B or x2.shape[1] != H or x2.shape[3] != D or x2.dtype != x.dtype:
            raise ValueError("x2 %s does not match x %s" % (tuple(x2.shape), tuple(x.shape)))
        y2 = torch.empty(tuple(x2.shape), dtype=torch.float8_e4m3fn, device=device)
        if x2.shape[2] > 0:
            a.S2 = x2.shape[2]
            a.x2, a.y2 = x2.data_ptr(), y2.data_ptr()
            a.x2_stride, a.y2_stride = _strides(x2), _strides(y2)
    if scale is not None:
        scale = scale.to(device=device, dtype=torch.float32).reshape(1).contiguous()
        a.scale_in = scale.data_ptr()
    a.x_stride, a.y_stride = _strides(x), _strides(y)
    stream = _stream(device)
    a.stream = stream
    need = 4 * max(4096, B * H)
    buf = _QUANT_SCRATCH.get((device, stream))
    if buf is None or buf.numel() < need:
        buf = torch.empty(need, dtype=torch.uint8, device=device)
        _QUANT_SCRATCH[(device, stream)] = buf
    a.scratch, a.scratch_bytes = buf.data_ptr(), buf.numel()
    with _on_device(device):
        _lib.check(_lib.lib().xdit_fp8_quant(ctypes.byref(a)))
    return (y, descale) if x2 is None else (y, y2, descale)


_NORM_MODES = {None: _lib.NORM_NONE, "none": _lib.NORM_NONE, "head": _lib.NORM_HEAD, "token": _lib.NORM_TOKEN}
_ROPE_MODES = {"interleaved": _lib.ROPE_INTERLEAVED, "split_half": _lib.ROPE_SPLIT_HALF, "wan": _lib.ROPE_WAN}


def _prologue_job(x, weight, eps, norm, rotary_emb, rope, rope_row0, rope_rows, out, keep):
    """Argument struct of one prologue job; tensors that must outlive the launch go to `keep`."""
    device = x.device
    _check4("x", x, device)
    B, H, S, D = x.shape
    if out is None:
        out = torch.empty((B, H, S, D), dtype=x.dtype, device=device)
    else:
        _check4("out", out, device)
        if tuple(out.shape) != (B, H, S, D) or out.dtype != x.dtype:
            raise ValueError("out has the wrong shape or dtype")
    if norm not in _NORM_MODES:
        raise ValueError("norm must be None, 'head' or 'token'")
    a = _lib.PrologueArgs()
    a.struct_size = ctypes.sizeof(_lib.PrologueArgs)
    a.dtype = _code(x.dtype)
    a.norm = _NORM_MODES[norm]
    a.B, a.H, a.D, a.S = B, H, D, S
    a.eps = float(eps)
    a.x, a.y = x.data_ptr(), out.data_ptr()
    a.x_stride, a.y_stride = _strides(x), _strides(out)
    if weight is not None and a.norm != _lib.NORM_NONE:
        n = D if a.norm == _lib.NORM_HEAD else H * D
        if weight.dtype != x.dtype or weight.numel() != n or weight.device != device:
            raise ValueError("weight must have %d entries of dtype %s on %s" % (n, x.dtype, device))
        weight = weight.reshape(-1).contiguous()
        keep.append(weight)
        a.weight = weight.data_ptr()
    if rotary_emb is not None:
        if rope not in _ROPE_MODES:
            raise ValueError("rope must be one of %s" % (sorted(_ROPE_MODES),))
        cos, sin = rotary_emb
        for name, t in (("cos", cos), ("sin", sin)):
            if t.dtype != torch.float32 or t.shape[-1] != D or t.device != device:
                raise ValueError("%s must be an fp32 tensor with a last dimension of %d on %s" % (name, D, device))
        cos = cos.reshape(-1, D)
        sin = sin.reshape(-1, D)
        if cos.stride(-1) != 1 or sin.stride(-1) != 1 or cos.stride(0) != sin.stride(0):
            cos, sin = cos.contiguous(), sin.contiguous()
        keep += [cos, sin]
        if rope_rows is None:
            rope_rows = min(cos.shape[0], S - rope_row0)
        if cos.shape[0] < rope_rows or sin.shape[0] < rope_rows:
            raise ValueError("the cos / sin tables hold %d rows, %d are needed" % (cos.shape[0], rope_rows))
        a.rope = _ROPE_MODES[rope]
        a.cos, a.sin = cos.data_ptr(), sin.data_ptr()
        a.rope_stride = cos.stride(0)
        a.rope_row0, a.rope_rows = int(rope_row0), int(rope_rows)
    a.stream = _stream(device)
    return a, out


def qk_prologue(x, weight=None, eps=1e-6, norm=None, rotary_emb=None, rope="interleaved",
                rope_row0=0, rope_rows=None, out=None):
    """RMSNorm + rotary embedding + re-layout of a logical BHSD tensor in one pass -> `out`
    (logical BHSD, any strides; a new BHSD-contiguous tensor when omitted).

    `norm`: None, "head" (over head_dim, `weight` has D entries) or "token" (over all heads of a
    token, `weight` has H*D entries); `weight` is in x's dtype or None.  `rotary_emb` = (cos, sin),
    fp32 tensors whose last dimension is D and whose rows (all other dimensions flattened) are the
    positions; rows [rope_row0, rope_row0 + rope_rows) of S are rotated with table row s - rope_row0.
    """
    keep = []
    a, out = _prologue_job(x, weight, eps, norm, rotary_emb, rope, rope_row0, rope_rows, out, keep)
    with _on_device(x.device):
        _lib.check(_lib.lib().xdit_qk_prologue(ctypes.byref(a)))
    return out


def prologue_batch_args(jobs):
    """The argument structs of up to 8 prologue jobs (dicts of the keyword arguments of
    `qk_prologue`, with `x`) as one ctypes array, for `launch_prologue_batch`; the outputs are in
    the jobs' `out` entries (created when missing).  The array keeps the tensors it points to alive
    only through the caller's own references."""
    if not 1 <= len(jobs) <= 8:
        raise ValueError("a batch holds 1 to 8 jobs")
    keep = []
    arr = (_lib.PrologueArgs * len(jobs))()
    for i, j in enumerate(jobs):
        a, out = _prologue_job(j["x"], j.get("weight"), j.get("eps", 1e-6), j.get("norm"), j.get("rotary_emb"),
                               j.get("rope", "interleaved"), j.get("rope_row0", 0), j.get("rope_rows"), j.get("out"), keep)
        arr[i] = a
        j["out"] = out
    arr._keep = keep
    return arr


def launch_prologue_batch(arr, count, device):
    """One launch of the first `count` jobs of an array from `prologue_batch_args` on the current
    stream of `device` (pointers may have been patched since)."""
    stream = _stream(device)
    for i in range(count):
        arr[i].stream = stream
    with _on_device(device):
        rc = _lib.lib().xdit_qk_prologue_batch(arr, count)
    if rc != 0:
        _lib.check(rc)


def qk_prologue_batch(jobs):
    """Up to 8 prologue jobs of one dtype on one device in ONE launch.  Each job is a dict of the
    keyword arguments of `qk_prologue` (with `x`).  Returns the list of outputs."""
    arr = prologue_batch_args(jobs)
    launch_prologue_batch(arr, len(jobs), jobs[0]["x"].device)
    return [j["out"] for j in jobs]
