"""MI355X-native attention hot path (joint-attention forward + ring LSE merge) behind
xDiT's attention call surfaces."""
from .ops import attn_fwd, attn_fwd_accumulate, fp8_quant, launch_plan, lse_merge  # noqa: F401
