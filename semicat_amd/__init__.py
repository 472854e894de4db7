"""MI355X-native fused attention-JVP: the ``sdpa_jvp`` / ``safe_sdpa_jvp`` op of olsdavis/semicat
(semicat/jvp_utils/functional.py) on hand-written gfx950 HIP kernels."""
from .functional import (SDPAFunction, SDPAJVPForwardFunction, SDPAJVPFlashBackwardFunction,
                         SDPABackwardFunction, SDPAFusedFunction, SDPAPrimalFunction, safe_sdpa_jvp,
                         safe_sdpa_jvp_rotary, sdpa_jvp)
from .kernels import (attention_forward, attention_jvp_backward, attention_jvp_forward,
                      flash_attention_jvp_multihead_kernel_wrapper, flash_attn_backward,
                      flash_jvp_backward)

__all__ = [
    "sdpa_jvp", "safe_sdpa_jvp", "safe_sdpa_jvp_rotary", "SDPAFusedFunction", "SDPAFunction", "SDPAJVPForwardFunction",
    "SDPAJVPFlashBackwardFunction", "SDPABackwardFunction", "SDPAPrimalFunction",
    "attention_forward", "attention_jvp_forward", "attention_jvp_backward",
    "flash_attention_jvp_multihead_kernel_wrapper", "flash_jvp_backward", "flash_attn_backward",
]
