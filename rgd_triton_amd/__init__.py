"""MI355X (gfx950) implementation of the rgd-triton operator set: hand-written HIP kernels behind the
reference's torch.nn.Module / autograd.Function API.  No Triton, no CPU fallback."""
from .ops import (CachableModule, FlashAttention, FusedHeadLayerNorm, FusedL2Normalize2, FusedLNRoPE, FusedRMSNorm,
                  FusedRMSNorm2, L2Normalize, RoPE)
from .functional import (clear_bias_classes_cache, flash_attn_func, set_attention_backward, triton_fused_ln_func_fn, triton_fused_ln_rope_fn, triton_fused_norm_func_fn,
                         triton_fused_rms_func_fn, triton_norm_func_fn, triton_rms_func_fn, triton_rope_fn)

__version__ = "0.1.0"
