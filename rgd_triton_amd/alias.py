"""Optional import-path alias: after `rgd_triton_amd.alias.install()` the reference's import paths
resolve to this package, so user code and test bodies written against rgd-triton run unchanged:

    from rgd_triton.ops import FlashAttention, FusedRMSNorm
    from rgd_triton.triton.flash_attn.flash_attn_triton_cached import flash_attn_func
    from rgd_triton.triton.normalization.rmsnorm_cached import triton_rms_func_fn

Nothing is installed unless install() is called, and an already imported real `rgd_triton` is never
replaced."""
import sys
import types

from . import functional, ops

# reference module path (rgd_triton/triton/...) -> names it exports that this package provides
_MODULES = {
    "rgd_triton.triton.flash_attn.flash_attn_triton_cached": ["flash_attn_func", "FlashAttnFunc"],
    "rgd_triton.triton.normalization.rmsnorm_cached": ["triton_rms_func_fn", "RMS_Func"],
    "rgd_triton.triton.normalization.fused_rmsnorm_cached": ["triton_fused_rms_func_fn", "Fused_RMS_Func"],
    "rgd_triton.triton.normalization.head_layernorm_cached": ["triton_fused_ln_func_fn", "Fused_LNQK_Func"],
    "rgd_triton.triton.normalization.l2normalize_cached": ["triton_norm_func_fn", "Norm_Func"],
    "rgd_triton.triton.normalization.fused_l2normalize_cached": ["triton_fused_norm_func_fn", "Fused_Norm_Func"],
    "rgd_triton.triton.rope.head_rope_cached": ["triton_rope_fn", "CombinedRoPEFunc"],
    "rgd_triton.triton.rope.fused_ln_rope_cached": ["triton_fused_ln_rope_fn", "FusedRoPEFunc"],
}


def install():
    """Register `rgd_triton` and its submodules in sys.modules.  Returns the list of names registered."""
    if "rgd_triton" in sys.modules and not getattr(sys.modules["rgd_triton"], "__rgd_alias__", False):
        raise RuntimeError("a real rgd_triton package is already imported; not replacing it")
    made = []

    def mod(name):
        if name not in sys.modules:
            m = types.ModuleType(name)
            m.__rgd_alias__ = True
            m.__path__ = []  # mark as package so submodule imports resolve through sys.modules
            sys.modules[name] = m
            made.append(name)
            if "." in name:
                parent, child = name.rsplit(".", 1)
                setattr(mod(parent), child, m)
        return sys.modules[name]

    mod("rgd_triton")
    sys.modules["rgd_triton.ops"] = ops
    setattr(sys.modules["rgd_triton"], "ops", ops)
    made.append("rgd_triton.ops")
    for name, exported in _MODULES.items():
        m = mod(name)
        for sym in exported:
            setattr(m, sym, getattr(functional, sym))
    return made
