"""CPU-side checks of the boundary: the shared library loads, exports every symbol include/rgd_hip.h
declares, rejects bad arguments with an error code and a message before touching the GPU, and the
Python layer mirrors the reference's API surface.  No kernel is launched here."""
import ctypes
import inspect
import os

import pytest
import torch

from helpers import ROOT

from rgd_triton_amd import _hip


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_hip.LIB_PATH), "build with make -C rgd_triton_amd/csrc"
    lib = _hip.lib()
    declared = _hip.declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/rgd_hip.h but not exported"
        assert name in _hip._SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(_hip._SIGNATURES) == declared
    assert lib.rgd_version() == 3000 and lib.rgd_version() // 1000 == _hip.ABI_MAJOR
    assert lib.rgd_attn_seqlen_q_rounded(1) == 64 and lib.rgd_attn_seqlen_q_rounded(128) == 128
    assert lib.rgd_attn_seqlen_q_rounded(129) == 192
    # delta (required part) plus room for the partial sums of split workgroups
    assert lib.rgd_attn_bwd_workspace(2, 3, 100, 50, 64, 1) >= 2 * 3 * 128 * 4


def test_header_cites_the_reference_for_every_entry_point():
    text = open(os.path.join(ROOT, "include", "rgd_hip.h")).read()
    for fn in ("_rms_fwd", "_rms_bwd", "_fused_rms_fwd", "_fused_rms_bwd", "_norm_fwd", "_norm_bwd", "_fused_norm_fwd",
               "_fused_norm_bwd", "_fused_ln_qk_fwd", "_fused_ln_qk_bwd", "combined_rope_fn", "_fused_rope_ln_qk_fwd",
               "_fused_rope_ln_qk_bwd", "_flash_attn_forward", "_flash_attn_backward"):
        assert f"replaces {fn}," in text, fn


def test_error_paths_return_codes_without_a_gpu():
    lib = _hip.lib()
    t3 = _hip.Tensor3(0x1000, 64, 8)
    t4 = _hip.Tensor4(0x1000, 64, 8, 8)
    assert lib.rgd_rms_fwd(1, 1, 8, t3, t3, t3, 7, 0, 1e-6, None) == -1
    assert b"Only support fp16, bf16, and fp32" in lib.rgd_last_error()
    assert lib.rgd_rms_fwd(1, 1, 8, None, t3, t3, 0, 0, 1e-6, None) == -1
    assert lib.rgd_l2_fwd(70000, 1, 8, t3, t3, 0, 1e-6, None) == -1           # batch beyond the grid limit
    # the attention backward keeps offsets inside a staged tile in 32 bits: token strides of 2^24 elements are refused
    far = _hip.Tensor4(0x1000, 64, 8, 1 << 24)
    for pos in range(4):  # dout, q, k, v in turn
        args = [t4] * 5
        args[pos] = far
        assert lib.rgd_attn_bwd(1, 1, 8, 8, 64, *args, 0x1000, None, 0, 0, t4, t4, t4, None, 1, 0, 0.125, 1, None, 0x1000, 1 << 20,
                                None) == -2, pos
        assert b"token stride" in lib.rgd_last_error()
    assert lib.rgd_ln_qk_fwd(1, 1, 4, 4, 300, t4, t4, t4, t4, 0, 1e-6, None) == -1
    assert b"head dimensions up to 256" in lib.rgd_last_error()
    assert lib.rgd_rope_qk(1, 1, 4, 4, 160, t4, t4, t4, t4, 0x1000, 8, 32, 256, 32, 0, 4, 4, 0, 0, None) == -1
    assert b"head dimensions up to 128" in lib.rgd_last_error()
    assert lib.rgd_rope_qk(1, 1, 8, 8, 64, t4, t4, t4, t4, 0x1000, 8, 32, 256, 32, 0, 8, 8, 0, 0, None) == -1  # T < P
    assert lib.rgd_attn_fwd(1, 1, 8, 8, 64, t4, t4, t4, None, 0, 0, t4, 0x1000, 0, 0, 0.125, None, None, 0, None) == -1
    assert b"Only support fp16 and bf16" in lib.rgd_last_error()
    assert lib.rgd_attn_fwd(1, 1, 8, 8, 200, t4, t4, t4, None, 0, 0, t4, 0x1000, 1, 0, 0.125, None, None, 0, None) == -1
    assert b"head dimensions up to 128" in lib.rgd_last_error()
    assert lib.rgd_attn_fwd(1, 1, 8, 8, 64, t4, t4, t4, t4, 2, 2, t4, 0x1000, 1, 0, 0.125, None, None, 0, None) == -1  # bias dtype
    assert lib.rgd_attn_bwd(1, 1, 8, 8, 64, t4, t4, t4, t4, t4, 0x1000, None, 0, 0, t4, t4, t4, None, 1, 0, 0.125, 1, None, 0x1000, 16,
                            None) == -4
    # the one-pass form needs room for dq_accum behind delta, and exists for head dims up to 64
    assert lib.rgd_attn_bwd_workspace(1, 1, 8, 8, 64, 2) >= 64 * 4 + 64 * 64 * 4
    assert lib.rgd_attn_bwd(1, 1, 8, 8, 64, t4, t4, t4, t4, t4, 0x1000, None, 0, 0, t4, t4, t4, None, 1, 0, 0.125, 2, None, 0x1000, 1024,
                            None) == -4
    assert lib.rgd_attn_bwd(1, 1, 8, 8, 128, t4, t4, t4, t4, t4, 0x1000, None, 0, 0, t4, t4, t4, None, 1, 0, 0.125, 2, None, 0x1000,
                            1 << 20, None) == -2
    assert lib.rgd_attn_bwd(1, 1, 8, 8, 64, t4, t4, t4, t4, t4, 0x1000, None, 0, 0, t4, t4, t4, None, 1, 0, 0.125, 7, None, 0x1000,
                            1 << 20, None) == -1
    # zero-sized problems are a successful no-op
    assert lib.rgd_l2_fwd(0, 0, 8, t3, t3, 0, 1e-6, None) == 0
    # one fp32 partial dw row per block
    assert lib.rgd_rms_bwd_workspace(4, 1024, 1024, 0, 0) >= 256 * 1024 * 4
    # a too small workspace is refused before any launch
    assert lib.rgd_rms_bwd(4, 1024, 1024, t3, t3, t3, t3, t3, 1, 0, 0, 1e-6, 0x1000, 16, None) == -4


def test_set_up_does_not_latch_without_a_device():
    """Without a usable GPU rgd_init reports that and keeps nothing: the argument checks and workspace queries above still
    work afterwards, and a second call says the same again.  (With a GPU it returns 0 and the test ends there.)"""
    import torch

    lib = _hip.lib()
    rc = lib.rgd_init()
    if torch.cuda.is_available():
        assert rc == 0, lib.rgd_last_error()
        return
    assert rc == -3 and b"no usable device" in lib.rgd_last_error()
    assert lib.rgd_attn_bwd_workspace(1, 2, 64, 64, 64, 1) > 0 and lib.rgd_rms_bwd_workspace(4, 1024, 1024, 0, 0) > 0
    assert lib.rgd_init() == -3
    # tile classes: sizes are plain host arithmetic
    shared = _hip.Tensor4(0x1000, 64 * 128, 0, 128)
    n = lib.rgd_attn_bias_classes_bytes(2, 4, 64, 128, 64, shared, _hip.BIAS_MATRIX, 2)
    assert n > 0 and n % 8 == 0
    assert lib.rgd_attn_bias_classes_bytes(2, 4, 64, 128, 128, shared, _hip.BIAS_MATRIX, 2) == 0       # head dim above 64
    per_head = _hip.Tensor4(0x1000, 4 * 64 * 128, 64 * 128, 128)
    assert lib.rgd_attn_bias_classes_bytes(2, 4, 64, 128, 64, per_head, _hip.BIAS_MATRIX, 2) == 0     # not shared by the heads
    assert lib.rgd_attn_bias_classes_bytes(2, 4, 64, 128, 64, shared, _hip.BIAS_VECTOR, 2) == n       # a vector: the same map
    assert lib.rgd_attn_bias_classify(2, 4, 64, 128, 64, shared, _hip.BIAS_MATRIX, 2, 0x1000, 8, None) == -4
    assert b"classes" in lib.rgd_last_error()


def test_module_api_surface_matches_reference():
    import rgd_triton_amd as rgd

    def params(fn):
        return [(n, p.default) for n, p in inspect.signature(fn).parameters.items() if n != "self"]

    E = inspect.Parameter.empty
    assert params(rgd.FlashAttention.forward) == [("q", E), ("k", E), ("v", E), ("bias", None), ("causal", False), ("softmax_scale", None)]
    assert params(rgd.L2Normalize.forward) == [("x", E), ("eps", 1e-6)]
    assert params(rgd.FusedL2Normalize2.forward) == [("x1", E), ("x2", E), ("eps", 1e-6)]
    assert params(rgd.FusedHeadLayerNorm.forward) == [("query", E), ("key", E), ("heads_second", True), ("eps", 1e-6)]
    assert params(rgd.FusedRMSNorm.__init__) == [("normalized_shape", E), ("eps", 1e-6), ("elementwise_affine", True), ("device", None), ("dtype", None)]
    assert params(rgd.FusedRMSNorm.forward) == [("x", E), ("weight", None)]
    assert params(rgd.FusedRMSNorm2.forward) == [("x1", E), ("x2", E), ("weight1", None), ("weight2", None)]
    assert params(rgd.RoPE.forward) == [("query", E), ("key", E), ("pos_emb", E), ("seq_cutoff", None), ("heads_second", True)]
    assert params(rgd.FusedLNRoPE.forward) == [("query", E), ("key", E), ("pos_emb", E), ("seq_cutoff", None), ("heads_second", True), ("eps", 1e-6)]
    assert params(rgd.flash_attn_func) == [("q", E), ("k", E), ("v", E), ("bias", None), ("causal", False), ("softmax_scale", None), ("return_lse", False), ("kernel_cache", None)]
    assert params(rgd.triton_rms_func_fn) == [("x", E), ("w", E), ("norm_eps", 1e-6), ("kernel_cache", None)]
    assert params(rgd.triton_fused_rms_func_fn) == [("x1", E), ("x2", E), ("w1", E), ("w2", E), ("norm_eps", 1e-6), ("kernel_cache", None)]
    assert params(rgd.triton_fused_ln_func_fn) == [("query", E), ("key", E), ("heads_second", True), ("norm_eps", 1e-6), ("kernel_cache", None)]
    assert params(rgd.triton_norm_func_fn) == [("x", E), ("norm_eps", 1e-6), ("use_ptx", False), ("kernel_cache", None)]
    assert params(rgd.triton_fused_norm_func_fn) == [("x1", E), ("x2", E), ("norm_eps", 1e-6), ("kernel_cache", None)]
    assert params(rgd.triton_fused_ln_rope_fn) == [("query", E), ("key", E), ("pos_emb", E), ("seq_cutoff", None), ("heads_second", True), ("norm_eps", 1e-6), ("kernel_cache", None)]
    assert params(rgd.triton_rope_fn)[:7] == [("query", E), ("key", E), ("pos_emb", E), ("seq_cutoff", None), ("heads_second", True), ("fused_ln", False), ("kernel_cache", None)]


def test_cachable_module_and_parameters_on_cpu():
    import rgd_triton_amd as rgd

    fields = {rgd.FlashAttention: ("fwd", "bwd_odot", "bwd"), rgd.L2Normalize: ("fwd", "bwd"), rgd.RoPE: ("fwd", "bwd"),
              rgd.FusedLNRoPE: ("fwd", "bwd"), rgd.FusedHeadLayerNorm: ("fwd", "bwd"), rgd.FusedL2Normalize2: ("fwd", "bwd")}
    for cls, names in fields.items():
        m = cls()
        assert all(getattr(m.cache, n, "missing") is None for n in names)
        m.enable_cache(False)
        assert m.cache is None
        m.enable_cache()
        assert m.cache is not None and getattr(m.cache, names[0]) is None
        assert len(list(m.parameters())) == 0
    m = rgd.FusedRMSNorm(48, eps=1e-5)
    assert m.normalized_shape == (48,) and m.eps == 1e-5 and m.weight.shape == (48,) and torch.all(m.weight == 1)
    m2 = rgd.FusedRMSNorm2([48, 16], dtype=torch.bfloat16)
    assert m2.normalized_shape1 == (48,) and m2.normalized_shape2 == (16,) and m2.weight2.dtype == torch.bfloat16
    sd = m2.state_dict()
    m3 = rgd.FusedRMSNorm2((48, 16), dtype=torch.bfloat16)
    m3.load_state_dict(sd)
    assert rgd.FusedRMSNorm(8, elementwise_affine=False).weight is None


def test_operators_refuse_cpu_tensors():
    """there is no CPU fallback: CPU tensors are rejected loudly"""
    import rgd_triton_amd as rgd

    x = torch.randn(2, 4, 16)
    with pytest.raises(AssertionError):
        rgd.L2Normalize()(x)
    with pytest.raises(AssertionError):
        rgd.FusedRMSNorm(16)(x)
    q = torch.randn(1, 2, 4, 16)
    with pytest.raises(AssertionError):
        rgd.FusedHeadLayerNorm()(q, q)
    with pytest.raises(AssertionError):
        rgd.FlashAttention()(q.half(), q.half(), q.half())


def test_reference_import_paths_alias():
    """rgd_triton_amd.alias.install() makes the reference's import paths resolve to this package"""
    import importlib
    import sys

    from rgd_triton_amd import alias

    assert "rgd_triton" not in sys.modules
    try:
        names = alias.install()
        assert "rgd_triton.ops" in names
        from rgd_triton.ops import FlashAttention, FusedRMSNorm2  # noqa: F401
        from rgd_triton.triton.flash_attn.flash_attn_triton_cached import flash_attn_func
        from rgd_triton.triton.normalization.fused_rmsnorm_cached import triton_fused_rms_func_fn
        from rgd_triton.triton.rope.fused_ln_rope_cached import triton_fused_ln_rope_fn
        import rgd_triton_amd as rgd

        assert flash_attn_func is rgd.flash_attn_func and triton_fused_rms_func_fn is rgd.triton_fused_rms_func_fn
        assert triton_fused_ln_rope_fn is rgd.triton_fused_ln_rope_fn and FlashAttention is rgd.FlashAttention
        assert importlib.import_module("rgd_triton.triton.rope.head_rope_cached").triton_rope_fn is rgd.triton_rope_fn
    finally:
        for k in [k for k in sys.modules if k == "rgd_triton" or k.startswith("rgd_triton.")]:
            del sys.modules[k]
