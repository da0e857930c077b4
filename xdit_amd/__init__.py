"""MI355X-native attention hot path (joint-attention forward + ring LSE merge) behind
xDiT's attention call surfaces."""
from .ops import attn_fwd, fp8_quant, lse_merge  # noqa: F401
