"""Single-device form of xDiT's legacy long-context attention path (BSHD tensors):
xfuser/core/long_ctx_attention/ring/ring_flash_attn.py and hybrid/attn_layer.py.

* `flash_attn_forward`            the per-step kernel call surface the ring loop uses
                                  (ring_flash_attn.py:107-134): BSHD in, (block_out BSHD,
                                  block_lse (B,H,Sq)) out.
* `update_out_and_lse`            the accumulator update called at ring_flash_attn.py:138.
* `xdit_ring_flash_attn_forward`  the loop of ring_flash_attn.py:27-148.  With no process group
                                  the ring has one member (the reference's single-GPU case); a
                                  `LocalRing(P)` runs the P-step schedule of one rank on one device.
* `xdit_ring_flash_attn_func`     defaults of ring_flash_attn.py:153-210, :248-312.
* `xFuserLongContextAttention`    the layer form, attn_layer.py:36-239, with the Ulysses
                                  all-to-alls being identities for a group of one.
"""
import math

import torch

from . import ops


class LocalRing:
    """Stand-in for a ring process group on one device: `world_size` KV chunks, visited in the
    order rank `rank` of a send-to-next / receive-from-previous ring would hold them
    (rank, rank-1, ..., mod world_size)."""

    def __init__(self, world_size, rank=0):
        if world_size < 1 or not (0 <= rank < world_size):
            raise ValueError("bad ring geometry")
        self.world_size = world_size
        self.rank = rank

    def order(self):
        return [(self.rank - s) % self.world_size for s in range(self.world_size)]


def _check_kernel_options(dropout_p, causal, window_size, softcap, alibi_slopes):
    if dropout_p not in (0, 0.0, None):
        raise ValueError(f"dropout_p={dropout_p} is not supported (must be 0.0)")
    if causal:
        raise NotImplementedError("causal=True is not implemented: DiT attention is non-causal")
    if tuple(window_size) != (-1, -1):
        raise NotImplementedError("sliding-window attention is not implemented")
    if softcap not in (0, 0.0, None):
        raise NotImplementedError("softcap is not implemented")
    if alibi_slopes is not None:
        raise NotImplementedError("alibi_slopes is not implemented")


def flash_attn_forward(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                       softcap=0.0, alibi_slopes=None, return_softmax=False, q_descale=None,
                       k_descale=None, v_descale=None, joint_k=None, joint_v=None, out_dtype=None):
    """Attention forward on BSHD tensors -> (block_out (B,Sq,H,D), block_lse (B,H,Sq) fp32).
    `joint_k`/`joint_v` (BSHD) are a second KV segment appended after `k`/`v`."""
    _check_kernel_options(dropout_p, causal, window_size, softcap, alibi_slopes)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.size(-1))
    t = lambda x: None if x is None else x.transpose(1, 2)  # BSHD -> logical BHSD view, no copy
    B, Sq, H, D = q.shape
    if out_dtype is None:
        out_dtype = torch.bfloat16 if q.dtype == torch.float8_e4m3fn else q.dtype
    out = torch.empty((B, Sq, H, D), dtype=out_dtype, device=q.device)
    _, lse = ops.attn_fwd(t(q), t(k), t(v), softmax_scale=softmax_scale, k2=t(joint_k), v2=t(joint_v),
                          q_descale=q_descale, k_descale=k_descale, v_descale=v_descale,
                          out_dtype=out_dtype, out=out.transpose(1, 2))
    return out, lse


def update_out_and_lse(out, lse, block_out, block_lse, slice_=None, final_out=None):
    """Accumulator update of the ring loop.  block_out (B,S,H,D), block_lse (B,H,S) fp32;
    accumulator `out` fp32 (B,S,H,D) and `lse` fp32 (B,S,H,1).  The first call (out is None)
    creates the accumulator from the block.  `final_out`, if given, also receives the merged rows
    cast to its dtype (fusing the `out.to(q.dtype)` epilogue)."""
    if slice_ is not None:
        raise NotImplementedError("slice_ is not supported (xDiT never passes it)")
    B, S, H, D = block_out.shape
    first = out is None
    if first:
        if lse is not None:
            raise ValueError("out and lse should be None or not None simultaneously.")
        out = torch.empty((B, S, H, D), dtype=torch.float32, device=block_out.device)
        lse = torch.empty((B, S, H, 1), dtype=torch.float32, device=block_out.device)
    ops.lse_merge(out.transpose(1, 2), lse.squeeze(-1).transpose(1, 2), block_out.transpose(1, 2), block_lse,
                  first=first, final_out=None if final_out is None else final_out.transpose(1, 2))
    return out, lse


def xdit_ring_flash_attn_forward(process_group, q, k, v, softmax_scale, dropout_p=0, causal=True,
                                 window_size=(-1, -1), alibi_slopes=None, deterministic=False,
                                 attn_type=None, attn_processor=None, attn_layer=None,
                                 joint_tensor_key=None, joint_tensor_value=None, joint_strategy="none",
                                 q_descale=None, k_descale=None, v_descale=None):
    """The ring loop on one device (ring_flash_attn.py:27-148), BSHD tensors.

    process_group None        -> one step over all of k, v (the reference's single-GPU case).
    process_group LocalRing(P) -> k, v hold the FULL key/value sequence; they are split into P
                                 chunks visited in the order the ring would deliver them.
    Returns (out in q's dtype (bf16 for fp8 inputs), lse (B,H,Sq) fp32)."""
    is_joint = False
    if joint_tensor_key is not None and joint_tensor_value is not None:
        supported_joint_strategy = ["front", "rear"]
        if joint_strategy not in supported_joint_strategy:
            raise ValueError(
                f"joint_strategy: {joint_strategy} not supprted. supported joint strategy: {supported_joint_strategy}"
            )
        is_joint = True
    elif joint_tensor_key is None and joint_tensor_value is None:
        pass
    else:
        raise ValueError("joint_tensor_key and joint_tensor_value should be None or not None simultaneously.")
    if attn_layer is not None:
        raise NotImplementedError("attn_layer (PipeFusion KV cache) is not supported on the single-device path")
    if process_group is None:
        process_group = LocalRing(1)
    if not isinstance(process_group, LocalRing):
        raise NotImplementedError("only a single-device LocalRing is supported")
    P = process_group.world_size
    if k.shape[1] % P != 0:
        raise ValueError(f"key length {k.shape[1]} is not divisible by the ring size {P}")
    k_chunks = k.chunk(P, dim=1)
    v_chunks = v.chunk(P, dim=1)
    out_dtype = torch.bfloat16 if q.dtype == torch.float8_e4m3fn else q.dtype

    out = None
    lse = None
    final = None
    # head_dim up to 128 (fp8: 128 or 64): every step is one launch that folds its block into the
    # accumulator in the kernel's epilogue (same bits as kernel call + update_out_and_lse).
    fused = P > 1 and ops.fused_ring_step_supported(q)
    t = lambda x: None if x is None else x.transpose(1, 2)
    for step, c in enumerate(process_group.order()):
        key, value = k_chunks[c], v_chunks[c]
        jk = jv = None
        if is_joint and ((joint_strategy == "rear" and step + 1 == P) or (joint_strategy == "front" and step == 0)):
            if joint_strategy == "rear":
                jk, jv = joint_tensor_key, joint_tensor_value
            else:  # "front": the joint tokens come first
                key, value, jk, jv = joint_tensor_key, joint_tensor_value, key, value
        if fused:
            _check_kernel_options(dropout_p, causal and step == 0, window_size, 0.0, alibi_slopes)
            B, Sq, H, D = q.shape
            if out is None:
                out = torch.empty((B, Sq, H, D), dtype=torch.float32, device=q.device)
                lse = torch.empty((B, Sq, H, 1), dtype=torch.float32, device=q.device)
            last = step + 1 == P
            if last:
                final = torch.empty((B, Sq, H, D), dtype=out_dtype, device=q.device)
            ops.attn_fwd_accumulate(t(q), t(key), t(value), t(out), lse.squeeze(-1).transpose(1, 2), first=step == 0,
                                    final_out=t(final), discard_acc_out=last, softmax_scale=softmax_scale,
                                    k2=t(jk), v2=t(jv), q_descale=q_descale, k_descale=k_descale,
                                    v_descale=v_descale, out_dtype=out_dtype)
            continue
        block_out, block_lse = flash_attn_forward(
            q, key, value, dropout_p=dropout_p, softmax_scale=softmax_scale, causal=causal and step == 0,
            window_size=window_size, softcap=0.0, alibi_slopes=alibi_slopes, return_softmax=False,
            q_descale=q_descale, k_descale=k_descale, v_descale=v_descale, joint_k=jk, joint_v=jv,
            out_dtype=out_dtype)
        if P == 1:
            # one step: the fold is the identity and the epilogue cast returns the block itself
            return block_out, block_lse
        if step + 1 == P:
            final = torch.empty_like(block_out)
        out, lse = update_out_and_lse(out, lse, block_out, block_lse, final_out=final)
    lse = lse.squeeze(dim=-1).transpose(1, 2)
    return final, lse


def xdit_ring_flash_attn_func(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                              alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None,
                              attn_type=None, attn_processor=None, attn_layer=None, joint_tensor_key=None,
                              joint_tensor_value=None, joint_strategy="none", q_descale=None, k_descale=None,
                              v_descale=None):
    """Forward-only counterpart of xdit_ring_flash_attn_func / xFuserRingFlashAttnFunc.forward
    (ring_flash_attn.py:153-210, :248-312): default scale 1/sqrt(D), `alibi_slopes` must be None,
    returns `out` or `(out, lse, None)` when `return_attn_probs`."""
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    assert alibi_slopes is None
    out, softmax_lse = xdit_ring_flash_attn_forward(
        group, q, k, v, softmax_scale=softmax_scale, dropout_p=dropout_p, causal=causal, window_size=window_size,
        alibi_slopes=alibi_slopes, deterministic=False, attn_type=attn_type, attn_processor=attn_processor,
        attn_layer=attn_layer, joint_tensor_key=joint_tensor_key, joint_tensor_value=joint_tensor_value,
        joint_strategy=joint_strategy, q_descale=q_descale, k_descale=k_descale, v_descale=v_descale)
    return out if not return_attn_probs else (out, softmax_lse, None)


class xFuserLongContextAttention(torch.nn.Module):
    """Layer form (attn_layer.py:36-239) for one device: BSHD in, BSHD out.  The Ulysses group has
    one member, so the head slice of the joint tensors (attn_layer.py:160-179) keeps every head
    and the SeqAllToAll4D exchanges (:183-202, :234-236) are identities."""

    def __init__(self, scatter_idx=2, gather_idx=1, ring_impl_type="basic", use_pack_qkv=False,
                 use_kv_cache=False, use_sync=False, attn_type=None, attn_processor=None,
                 q_descale=None, k_descale=None, v_descale=None, ring_group=None):
        super().__init__()
        if ring_impl_type != "basic":
            raise RuntimeError(f"ring_impl_type: {ring_impl_type} is not supported.")
        if use_kv_cache:
            raise NotImplementedError("use_kv_cache (PipeFusion) is not supported on the single-device path")
        self.scatter_idx = scatter_idx
        self.gather_idx = gather_idx
        self.use_pack_qkv = use_pack_qkv
        self.attn_type = attn_type
        self.attn_processor = attn_processor
        self.q_descale = q_descale
        self.k_descale = k_descale
        self.v_descale = v_descale
        self.ring_pg = ring_group
        self.ring_attn_fn = xdit_ring_flash_attn_func

    def forward(self, attn, query, key, value, *, joint_tensor_query=None, joint_tensor_key=None,
                joint_tensor_value=None, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                alibi_slopes=None, deterministic=False, return_attn_probs=False, joint_strategy="none"):
        if joint_tensor_query is not None and joint_tensor_key is not None and joint_tensor_value is not None:
            supported_joint_strategy = ["front", "rear"]
            if joint_strategy not in supported_joint_strategy:
                raise ValueError(
                    f"joint_strategy: {joint_strategy} not supprted. supported joint strategy: {supported_joint_strategy}"
                )
            elif joint_strategy == "rear":
                query = torch.cat([query, joint_tensor_query], dim=1)
            else:
                query = torch.cat([joint_tensor_query, query], dim=1)
        elif joint_tensor_query is None and joint_tensor_key is None and joint_tensor_value is None:
            pass
        else:
            raise ValueError(
                "joint_tensor_query, joint_tensor_key, and joint_tensor_value should be None or not None simultaneously."
            )
        out = self.ring_attn_fn(
            query, key, value, dropout_p=dropout_p, softmax_scale=softmax_scale, causal=causal,
            window_size=window_size, alibi_slopes=alibi_slopes, deterministic=deterministic,
            return_attn_probs=return_attn_probs, group=self.ring_pg, attn_type=self.attn_type,
            attn_processor=self.attn_processor, attn_layer=None, joint_tensor_key=joint_tensor_key,
            joint_tensor_value=joint_tensor_value, joint_strategy=joint_strategy,
            q_descale=self.q_descale, k_descale=self.k_descale, v_descale=self.v_descale)
        if type(out) == tuple:
            context_layer, _, _ = out
        else:
            context_layer = out
        return context_layer
