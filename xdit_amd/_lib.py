"""ctypes binding of the C ABI declared in include/xdit_amd_attn.h.

The shared library is built in-tree by `xdit_amd.build` (hipcc, gfx950).  Loading never
falls back to anything else: if the library is missing, `lib()` raises.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libxdit_amd_attn.so")
ABI_VERSION = 8

XDIT_OK = 0
XDIT_ERR_INVALID_ARG = -1
XDIT_ERR_UNSUPPORTED = -2
XDIT_ERR_LAUNCH = -3

DTYPE_BF16, DTYPE_FP16, DTYPE_FP32, DTYPE_FP8_E4M3FN = 0, 1, 2, 3


class Strides(ctypes.Structure):
    _fields_ = [("b", ctypes.c_int64), ("h", ctypes.c_int64), ("s", ctypes.c_int64)]


class AttnArgs(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("causal", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("rows_per_workgroup", ctypes.c_int32),
        ("Sq", ctypes.c_int64),
        ("Sk", ctypes.c_int64),
        ("Sk2", ctypes.c_int64),
        ("softmax_scale", ctypes.c_float),
        ("cu_count", ctypes.c_int32),
        ("streamed_sharing", ctypes.c_int32),
        ("workspace_preserved", ctypes.c_int32),
        ("balance", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("k2", ctypes.c_void_p),
        ("v2", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("q_stride", Strides),
        ("k_stride", Strides),
        ("v_stride", Strides),
        ("k2_stride", Strides),
        ("v2_stride", Strides),
        ("out_stride", Strides),
        ("lse_stride_b", ctypes.c_int64),
        ("lse_stride_h", ctypes.c_int64),
        ("q_descale", ctypes.c_void_p),
        ("k_descale", ctypes.c_void_p),
        ("v_descale", ctypes.c_void_p),
        ("descale_stride_b", ctypes.c_int64),
        ("descale_stride_h", ctypes.c_int64),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_int64),
        ("stream", ctypes.c_void_p),
    ]


class MergeArgs(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("block_dtype", ctypes.c_int32),
        ("final_dtype", ctypes.c_int32),
        ("first", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
        ("S", ctypes.c_int64),
        ("acc_out", ctypes.c_void_p),
        ("acc_lse", ctypes.c_void_p),
        ("block_out", ctypes.c_void_p),
        ("block_lse", ctypes.c_void_p),
        ("final_out", ctypes.c_void_p),
        ("acc_out_stride", Strides),
        ("block_out_stride", Strides),
        ("final_out_stride", Strides),
        ("acc_lse_stride", Strides),
        ("block_lse_stride", Strides),
        ("stream", ctypes.c_void_p),
    ]


class LaunchPlan(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("rows_per_workgroup", ctypes.c_int32),
        ("query_tiles", ctypes.c_int32),
        ("kv_iterations", ctypes.c_int32),
        ("workspace_bytes", ctypes.c_int64),
        ("whole_tiles", ctypes.c_int32),
        ("ranges", ctypes.c_int32),
        ("range_len", ctypes.c_int32),
        ("slots_per_tile", ctypes.c_int32),
        ("claimers", ctypes.c_int32),
        ("first_claimer", ctypes.c_int32),
        ("counter", ctypes.c_int32),
        ("workgroups", ctypes.c_int32),
        ("streamed", ctypes.c_int32),
        ("fold_in_kernel", ctypes.c_int32),
        ("parts_first", ctypes.c_int32),
        ("ring_step", ctypes.c_int32),
    ]


class RingAcc(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("first", ctypes.c_int32),
        ("discard_acc_out", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
        ("acc_out", ctypes.c_void_p),
        ("acc_lse", ctypes.c_void_p),
        ("acc_out_stride", Strides),
        ("acc_lse_stride", Strides),
    ]


class QuantArgs(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("in_dtype", ctypes.c_int32),
        ("per_tensor", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("S", ctypes.c_int64),
        ("x", ctypes.c_void_p),
        ("y", ctypes.c_void_p),
        ("descale", ctypes.c_void_p),
        ("scale_in", ctypes.c_void_p),
        ("x_stride", Strides),
        ("y_stride", Strides),
        ("stream", ctypes.c_void_p),
        ("hadamard_block", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
        ("S2", ctypes.c_int64),
        ("x2", ctypes.c_void_p),
        ("y2", ctypes.c_void_p),
        ("x2_stride", Strides),
        ("y2_stride", Strides),
        ("scratch", ctypes.c_void_p),
        ("scratch_bytes", ctypes.c_int64),
    ]


class PrologueArgs(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("norm", ctypes.c_int32),
        ("rope", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("eps", ctypes.c_float),
        ("S", ctypes.c_int64),
        ("x", ctypes.c_void_p),
        ("y", ctypes.c_void_p),
        ("weight", ctypes.c_void_p),
        ("cos", ctypes.c_void_p),
        ("sin", ctypes.c_void_p),
        ("rope_stride", ctypes.c_int64),
        ("rope_row0", ctypes.c_int64),
        ("rope_rows", ctypes.c_int64),
        ("x_stride", Strides),
        ("y_stride", Strides),
        ("stream", ctypes.c_void_p),
    ]


NORM_NONE, NORM_HEAD, NORM_TOKEN = 0, 1, 2
ROPE_NONE, ROPE_INTERLEAVED, ROPE_SPLIT_HALF, ROPE_WAN = 0, 1, 2, 3

EXPORTS = ("xdit_attn_fwd", "xdit_attn_fwd_noalloc", "xdit_attn_fwd_accumulate", "xdit_attn_workspace_bytes", "xdit_attn_launch_plan", "xdit_lse_merge", "xdit_fp8_quant", "xdit_qk_prologue", "xdit_qk_prologue_batch", "xdit_attn_last_error", "xdit_attn_abi_version")

_lib = None
_lock = threading.Lock()


def lib():
    """Return the loaded shared library (loading it on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m xdit_amd.build` (hipcc, gfx950). "
                "There is no fallback path." % LIB_PATH
            )
        L = ctypes.CDLL(LIB_PATH)
        L.xdit_attn_fwd.argtypes = [ctypes.POINTER(AttnArgs)]
        L.xdit_attn_fwd.restype = ctypes.c_int
        L.xdit_attn_fwd_noalloc.argtypes = [ctypes.POINTER(AttnArgs)]
        L.xdit_attn_fwd_noalloc.restype = ctypes.c_int
        L.xdit_attn_fwd_accumulate.argtypes = [ctypes.POINTER(AttnArgs), ctypes.POINTER(RingAcc)]
        L.xdit_attn_fwd_accumulate.restype = ctypes.c_int
        L.xdit_attn_launch_plan.argtypes = [ctypes.POINTER(AttnArgs), ctypes.POINTER(LaunchPlan)]
        L.xdit_attn_launch_plan.restype = ctypes.c_int
        L.xdit_attn_workspace_bytes.argtypes = [ctypes.POINTER(AttnArgs)]
        L.xdit_attn_workspace_bytes.restype = ctypes.c_int64
        L.xdit_lse_merge.argtypes = [ctypes.POINTER(MergeArgs)]
        L.xdit_lse_merge.restype = ctypes.c_int
        L.xdit_fp8_quant.argtypes = [ctypes.POINTER(QuantArgs)]
        L.xdit_fp8_quant.restype = ctypes.c_int
        L.xdit_qk_prologue.argtypes = [ctypes.POINTER(PrologueArgs)]
        L.xdit_qk_prologue.restype = ctypes.c_int
        L.xdit_qk_prologue_batch.argtypes = [ctypes.POINTER(PrologueArgs), ctypes.c_int32]
        L.xdit_qk_prologue_batch.restype = ctypes.c_int
        L.xdit_attn_last_error.argtypes = []
        L.xdit_attn_last_error.restype = ctypes.c_char_p
        L.xdit_attn_abi_version.argtypes = []
        L.xdit_attn_abi_version.restype = ctypes.c_int
        v = L.xdit_attn_abi_version()
        if v != ABI_VERSION:
            raise RuntimeError("ABI version %d of %s != binding version %d" % (v, LIB_PATH, ABI_VERSION))
        _lib = L
    return _lib


def last_error():
    return lib().xdit_attn_last_error().decode("utf-8", "replace")


def check(rc):
    """Map a C status to the Python exception the reference's style uses:
    ValueError for argument errors, NotImplementedError for unsupported options,
    RuntimeError for launch failures."""
    if rc == XDIT_OK:
        return
    msg = last_error()
    if rc == XDIT_ERR_INVALID_ARG:
        raise ValueError(msg)
    if rc == XDIT_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
