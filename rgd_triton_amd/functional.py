"""torch.autograd.Function layer: the same functions, argument order and error behaviour as the
reference's `*_cached.py` modules, launching the gfx950 HIP kernels of librgd_hip.so through ctypes.

Reference entry points mirrored here (paths relative to rgd_triton/triton/):
    flash_attn_func            flash_attn/flash_attn_triton_cached.py:1079-1133
    triton_rms_func_fn         normalization/rmsnorm_cached.py:572-629
    triton_fused_rms_func_fn   normalization/fused_rmsnorm_cached.py:725-802
    triton_fused_ln_func_fn    normalization/head_layernorm_cached.py:416-457
    triton_norm_func_fn        normalization/l2normalize_cached.py:402-437
    triton_fused_norm_func_fn  normalization/fused_l2normalize_cached.py:464-507
    triton_rope_fn             rope/head_rope_cached.py:277-327
    triton_fused_ln_rope_fn    rope/fused_ln_rope_cached.py:649-696

Differences from the reference, all deliberate:
  * row statistics (rrms, mean/rstd, rlen) are recomputed in the backward instead of being saved;
  * dw of a shared RMSNorm weight is reduced in fp32 inside the kernel and rounded once;
  * `kernel_cache` objects keep their field names; a field holds the set of validated call
    signatures instead of a compiled-kernel handle, so a change of shape, dtype or bias kind after
    the first call can never reuse a stale specialisation.
"""
import ctypes
import math
import os

import torch

from . import _hip
from ._hip import t3, t4

__all__ = [
    "flash_attn_func", "triton_rms_func_fn", "triton_fused_rms_func_fn", "triton_fused_ln_func_fn",
    "triton_norm_func_fn", "triton_fused_norm_func_fn", "triton_rope_fn", "triton_fused_ln_rope_fn",
    "set_attention_backward",
]

_FLOATS = (torch.float16, torch.bfloat16, torch.float32)


def _lastdim_contig(*ts):
    return [t if (t is None or t.stride(-1) == 1) else t.contiguous() for t in ts]


def _seen(cache, field, key):
    """True if this call signature already went through validation with this cache object."""
    if cache is None:
        return False
    plans = getattr(cache, field, None)
    if plans is None:
        plans = set()
        setattr(cache, field, plans)
    if key in plans:
        return True
    plans.add(key)
    return False


def _no_capture(what):
    """Every backward starts here.  Recording an autograd backward of these operators into a HIP graph ended in a
    crash inside the runtime's end-of-capture call on the one occasion it was tried (the backward nodes run on
    autograd's worker thread), and its cause was never established, so the combination is refused with an error
    instead: record the backward through direct C-ABI calls (tests/test_graph_capture.py does) or keep autograd
    outside the graph.  The forward functions can be captured."""
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError(f"{what}: an autograd backward cannot be recorded into a HIP graph with this package; "
                           "record direct calls of the C ABI instead")


def _sig(*ts):
    return tuple((tuple(t.shape), t.dtype, tuple(t.stride())) if t is not None else None for t in ts)


# ----------------------------------------------------------------------------------------------
# RMSNorm
# ----------------------------------------------------------------------------------------------


def _w_layout(w, x):
    """Weight broadcast rule of the reference (rmsnorm_cached.py:582-589): returns (shared, stride_b)."""
    if w.ndim == 1:
        assert w.shape[0] == x.shape[-1], f"{x.shape=}, {w.shape=}"
        return True, 0
    assert w.ndim == 3 and w.shape[1] == 1 and w.shape[2] == x.shape[-1], f"{x.shape=}, {w.shape=}"
    if w.shape[0] == 1:
        return True, 0
    assert w.shape[0] == x.shape[0], f"{x.shape=}, {w.shape=}"
    return False, w.stride(0)


def _check_rows(x):
    assert x.ndim == 3, f"{x.shape=}"
    assert x.dtype in _FLOATS, "Only support fp16, bf16, and fp32"
    assert x.is_cuda, "rgd_triton_amd operators run on the GPU only"


def _rms_scratch(x1, x2):
    B = x1.shape[0]
    T2, C2 = (x2.shape[1], x2.shape[2]) if x2 is not None else (0, 0)
    nbytes = _hip.lib().rgd_rms_bwd_workspace(B, x1.shape[1], x1.shape[2], T2, C2)
    return _hip.workspace(x1.device, nbytes), nbytes


class RMS_Func(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, norm_eps=1e-6, kernel_cache=None):
        x, w = _lastdim_contig(x, w)
        if not _seen(kernel_cache, "fwd", _sig(x, w)):
            _check_rows(x)
            assert w.is_cuda and w.dtype in _FLOATS, "Only support fp16, bf16, and fp32"
        shared, w_sb = _w_layout(w, x)
        B, T, C = x.shape
        y = torch.empty_like(x)
        lib = _hip.lib()
        _hip.check(lib.rgd_rms_fwd(B, T, C, t3(x), t3(w, w_sb), t3(y), _hip.dtype_code(x.dtype),
                                   _hip.dtype_code(w.dtype), float(norm_eps), _hip.stream_ptr(x.device)), "rgd_rms_fwd")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(x, w)
        ctx.norm_eps = float(norm_eps)
        ctx.w_layout = (shared, w_sb)
        return y

    @staticmethod
    def backward(ctx, dy):
        _no_capture("RMS_Func.backward")
        (dy,) = _lastdim_contig(dy)
        x, w = ctx.saved_tensors
        shared, w_sb = ctx.w_layout
        B, T, C = x.shape
        _seen(ctx.kernel_cache, "bwd", _sig(x, w, dy))
        _seen(ctx.kernel_cache, "bwd_dw", _sig(w))
        dx = torch.empty_like(x)
        dw = torch.empty(w.shape, dtype=w.dtype, device=w.device)
        if B * T == 0:
            dw.zero_()
            return dx, dw, None, None
        wbuf, wsz = _rms_scratch(x, None)
        lib = _hip.lib()
        _hip.check(lib.rgd_rms_bwd(B, T, C, t3(dy), t3(x), t3(w, w_sb), t3(dx), t3(dw, 0 if shared else dw.stride(0)),
                                   int(shared), _hip.dtype_code(x.dtype), _hip.dtype_code(w.dtype), ctx.norm_eps,
                                   wbuf.data_ptr(), wsz, _hip.stream_ptr(x.device)), "rgd_rms_bwd")
        return dx, dw, None, None


def triton_rms_func_fn(x, w, norm_eps=1e-6, kernel_cache=None):
    return RMS_Func.apply(x, w, norm_eps, kernel_cache)


class Fused_RMS_Func(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, w1, w2, norm_eps=1e-6, kernel_cache=None):
        x1, x2, w1, w2 = _lastdim_contig(x1, x2, w1, w2)
        if not _seen(kernel_cache, "fwd", _sig(x1, x2, w1, w2)):
            _check_rows(x1)
            _check_rows(x2)
            assert x1.dtype == x2.dtype, "All tensors must have the same type"
            assert x1.shape[0] == x2.shape[0], f"{x1.shape=}, {x2.shape=}"
            assert w1.is_cuda and w2.is_cuda and w1.dtype in _FLOATS and w2.dtype in _FLOATS
        l1, l2 = _w_layout(w1, x1), _w_layout(w2, x2)
        B, T1, C1 = x1.shape
        _, T2, C2 = x2.shape
        y1, y2 = torch.empty_like(x1), torch.empty_like(x2)
        lib = _hip.lib()
        _hip.check(lib.rgd_fused_rms_fwd(B, T1, C1, T2, C2, t3(x1), t3(w1, l1[1]), t3(y1), t3(x2), t3(w2, l2[1]), t3(y2),
                                         _hip.dtype_code(x1.dtype), _hip.dtype_code(w1.dtype), _hip.dtype_code(w2.dtype),
                                         float(norm_eps), _hip.stream_ptr(x1.device)), "rgd_fused_rms_fwd")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(x1, x2, w1, w2)
        ctx.norm_eps = float(norm_eps)
        ctx.layouts = (l1, l2)
        return y1, y2

    @staticmethod
    def backward(ctx, dy1, dy2):
        _no_capture("Fused_RMS_Func.backward")
        dy1, dy2 = _lastdim_contig(dy1, dy2)
        x1, x2, w1, w2 = ctx.saved_tensors
        (s1, sb1), (s2, sb2) = ctx.layouts
        B, T1, C1 = x1.shape
        _, T2, C2 = x2.shape
        _seen(ctx.kernel_cache, "bwd", _sig(x1, x2, w1, w2, dy1, dy2))
        _seen(ctx.kernel_cache, "bwd_dw", _sig(w1, w2))
        dx1, dx2 = torch.empty_like(x1), torch.empty_like(x2)
        dw1 = torch.empty(w1.shape, dtype=w1.dtype, device=w1.device)
        dw2 = torch.empty(w2.shape, dtype=w2.dtype, device=w2.device)
        if B * T1 == 0:
            dw1.zero_()
        if B * T2 == 0:
            dw2.zero_()
        wbuf, wsz = _rms_scratch(x1, x2)
        lib = _hip.lib()
        _hip.check(lib.rgd_fused_rms_bwd(
            B, T1, C1, T2, C2,
            t3(dy1), t3(x1), t3(w1, sb1), t3(dx1), t3(dw1, 0 if s1 else dw1.stride(0)), int(s1),
            t3(dy2), t3(x2), t3(w2, sb2), t3(dx2), t3(dw2, 0 if s2 else dw2.stride(0)), int(s2),
            _hip.dtype_code(x1.dtype), _hip.dtype_code(w1.dtype), _hip.dtype_code(w2.dtype), ctx.norm_eps,
            wbuf.data_ptr(), wsz, _hip.stream_ptr(x1.device)), "rgd_fused_rms_bwd")
        return dx1, dx2, dw1, dw2, None, None


def triton_fused_rms_func_fn(x1, x2, w1, w2, norm_eps=1e-6, kernel_cache=None):
    return Fused_RMS_Func.apply(x1, x2, w1, w2, norm_eps, kernel_cache)


# ----------------------------------------------------------------------------------------------
# L2 normalize
# ----------------------------------------------------------------------------------------------


class Norm_Func(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, norm_eps=1e-6, use_ptx=False, kernel_cache=None):
        (x,) = _lastdim_contig(x)
        if not _seen(kernel_cache, "fwd", _sig(x)):
            _check_rows(x)
        B, T, C = x.shape
        y = torch.empty_like(x)
        lib = _hip.lib()
        _hip.check(lib.rgd_l2_fwd(B, T, C, t3(x), t3(y), _hip.dtype_code(x.dtype), float(norm_eps),
                                  _hip.stream_ptr(x.device)), "rgd_l2_fwd")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(x)
        ctx.norm_eps = float(norm_eps)
        return y

    @staticmethod
    def backward(ctx, dy):
        _no_capture("Norm_Func.backward")
        (dy,) = _lastdim_contig(dy)
        (x,) = ctx.saved_tensors
        B, T, C = x.shape
        _seen(ctx.kernel_cache, "bwd", _sig(x, dy))
        dx = torch.empty_like(x)
        lib = _hip.lib()
        _hip.check(lib.rgd_l2_bwd(B, T, C, t3(dy), t3(x), t3(dx), _hip.dtype_code(x.dtype), ctx.norm_eps,
                                  _hip.stream_ptr(x.device)), "rgd_l2_bwd")
        return dx, None, None, None


def triton_norm_func_fn(x, norm_eps=1e-6, use_ptx=False, kernel_cache=None):
    # use_ptx selected an NVIDIA inline-PTX reciprocal in the reference
    # (l2normalize_cached.py:79-98); it has no meaning here and is ignored
    return Norm_Func.apply(x, norm_eps, use_ptx, kernel_cache)


class Fused_Norm_Func(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, norm_eps=1e-6, kernel_cache=None):
        x1, x2 = _lastdim_contig(x1, x2)
        if not _seen(kernel_cache, "fwd", _sig(x1, x2)):
            _check_rows(x1)
            _check_rows(x2)
            assert x1.dtype == x2.dtype, "All tensors must have the same type"
            assert x1.shape[0] == x2.shape[0], f"{x1.shape=}, {x2.shape=}"
        B, T1, C1 = x1.shape
        _, T2, C2 = x2.shape
        y1, y2 = torch.empty_like(x1), torch.empty_like(x2)
        lib = _hip.lib()
        _hip.check(lib.rgd_fused_l2_fwd(B, T1, C1, T2, C2, t3(x1), t3(y1), t3(x2), t3(y2), _hip.dtype_code(x1.dtype),
                                        float(norm_eps), _hip.stream_ptr(x1.device)), "rgd_fused_l2_fwd")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(x1, x2)
        ctx.norm_eps = float(norm_eps)
        return y1, y2

    @staticmethod
    def backward(ctx, dy1, dy2):
        _no_capture("Fused_Norm_Func.backward")
        dy1, dy2 = _lastdim_contig(dy1, dy2)
        x1, x2 = ctx.saved_tensors
        B, T1, C1 = x1.shape
        _, T2, C2 = x2.shape
        _seen(ctx.kernel_cache, "bwd", _sig(x1, x2, dy1, dy2))
        dx1, dx2 = torch.empty_like(x1), torch.empty_like(x2)
        lib = _hip.lib()
        _hip.check(lib.rgd_fused_l2_bwd(B, T1, C1, T2, C2, t3(dy1), t3(x1), t3(dx1), t3(dy2), t3(x2), t3(dx2),
                                        _hip.dtype_code(x1.dtype), ctx.norm_eps, _hip.stream_ptr(x1.device)),
                   "rgd_fused_l2_bwd")
        return dx1, dx2, None, None


def triton_fused_norm_func_fn(x1, x2, norm_eps=1e-6, kernel_cache=None):
    return Fused_Norm_Func.apply(x1, x2, norm_eps, kernel_cache)


# ----------------------------------------------------------------------------------------------
# per-head operators on (query, key)
# ----------------------------------------------------------------------------------------------


def _qk_dims(q, k, heads_second, max_d, what):
    assert q.ndim == k.ndim == 4
    assert q.dtype == k.dtype, "All tensors must have the same type"
    assert q.dtype in _FLOATS, "Only support fp16, bf16, and fp32"
    assert q.is_cuda and k.is_cuda, "rgd_triton_amd operators run on the GPU only"
    if heads_second:
        bq, hq, tq, dq = q.shape
        bk, hk, tk, dk = k.shape
    else:
        bq, tq, hq, dq = q.shape
        bk, tk, hk, dk = k.shape
    assert (bq, hq, dq) == (bk, hk, dk)
    assert dq <= max_d, f"Only supports head dimensions up to {max_d}"
    return bq, hq, tq, tk, dq


def _cutoffs(seq_cutoff, tq, tk):
    # head_rope_cached.py:193-201
    if seq_cutoff is None:
        return tq, tk
    if isinstance(seq_cutoff, (tuple, list)):
        return int(seq_cutoff[0]), int(seq_cutoff[1])
    return int(seq_cutoff), int(seq_cutoff)


def _table_for(pos_emb, x):
    """A rotary table the kernels can read next to tensors of x.dtype: same dtype, or fp32."""
    if pos_emb.dtype == x.dtype or pos_emb.dtype == torch.float32:
        return pos_emb
    return pos_emb.float()  # e.g. an fp16 table with bf16 tensors: exact upcast, tiny tensor


def _pos_emb_args(pos_emb, tq, tk):
    """pos_emb (2, P, R) -> C arguments.  The kernels read a table in the tensors' dtype or in fp32; the
    caller has already converted any other combination (see _table_for)."""
    assert pos_emb.ndim == 3 and pos_emb.shape[0] == 2, f"{pos_emb.shape=}"
    assert pos_emb.is_cuda and pos_emb.dtype in _FLOATS
    _, P, R = pos_emb.shape
    assert tq < P
    assert tk < P
    return (ctypes.c_void_p(pos_emb.data_ptr()), P, R, pos_emb.stride(0), pos_emb.stride(1),
            _hip.dtype_code(pos_emb.dtype))


class Fused_LNQK_Func(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, heads_second=True, norm_eps=1e-6, kernel_cache=None):
        q, k = _lastdim_contig(q, k)
        _seen(kernel_cache, "fwd", _sig(q, k) + (heads_second,))
        B, H, Tq, Tk, D = _qk_dims(q, k, heads_second, 256, "head LayerNorm")
        qo, ko = torch.empty_like(q), torch.empty_like(k)
        lib = _hip.lib()
        _hip.check(lib.rgd_ln_qk_fwd(B, H, Tq, Tk, D, t4(q, heads_second), t4(k, heads_second), t4(qo, heads_second),
                                     t4(ko, heads_second), _hip.dtype_code(q.dtype), float(norm_eps),
                                     _hip.stream_ptr(q.device)), "rgd_ln_qk_fwd")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(q, k)
        ctx.heads_second = heads_second
        ctx.norm_eps = float(norm_eps)
        ctx.dims = (B, H, Tq, Tk, D)
        return qo, ko

    @staticmethod
    def backward(ctx, doq, dok):
        _no_capture("Fused_LNQK_Func.backward")
        q, k = ctx.saved_tensors
        hs = ctx.heads_second
        doq, dok = _lastdim_contig(doq, dok)
        _seen(ctx.kernel_cache, "bwd", _sig(q, k, doq, dok) + (hs,))
        B, H, Tq, Tk, D = ctx.dims
        dq, dk = torch.empty_like(q), torch.empty_like(k)
        lib = _hip.lib()
        _hip.check(lib.rgd_ln_qk_bwd(B, H, Tq, Tk, D, t4(q, hs), t4(k, hs), t4(doq, hs), t4(dok, hs), t4(dq, hs),
                                     t4(dk, hs), _hip.dtype_code(q.dtype), ctx.norm_eps, _hip.stream_ptr(q.device)),
                   "rgd_ln_qk_bwd")
        return dq, dk, None, None, None


def triton_fused_ln_func_fn(query, key, heads_second=True, norm_eps=1e-6, kernel_cache=None):
    return Fused_LNQK_Func.apply(query, key, heads_second, norm_eps, kernel_cache)


class CombinedRoPEFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, pos_emb, seq_cutoff=None, heads_second=True, in_place=False, kernel_cache=None):
        if in_place:
            assert q.stride(-1) == 1 and k.stride(-1) == 1, "in_place RoPE needs unit-stride head dims"
        q, k, pos_emb = _lastdim_contig(q, k, _table_for(pos_emb, q))
        _seen(kernel_cache, "fwd", _sig(q, k, pos_emb) + (heads_second,))
        B, H, Tq, Tk, D = _qk_dims(q, k, heads_second, 128, "RoPE")
        pe = _pos_emb_args(pos_emb, Tq, Tk)
        cq, ck = _cutoffs(seq_cutoff, Tq, Tk)
        if in_place:
            qo, ko = q, k
            ctx.mark_dirty(q, k)
        else:
            qo, ko = torch.empty_like(q), torch.empty_like(k)
        lib = _hip.lib()
        _hip.check(lib.rgd_rope_qk(B, H, Tq, Tk, D, t4(q, heads_second), t4(k, heads_second), t4(qo, heads_second),
                                   t4(ko, heads_second), *pe, cq, ck, 0, _hip.dtype_code(q.dtype),
                                   _hip.stream_ptr(q.device)), "rgd_rope_qk")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(pos_emb)
        ctx.seq_cutoff = (cq, ck)
        ctx.heads_second = heads_second
        ctx.dims = (B, H, Tq, Tk, D)
        return qo, ko

    @staticmethod
    def backward(ctx, doq, dok):
        _no_capture("CombinedRoPEFunc.backward")
        (pos_emb,) = ctx.saved_tensors
        assert not ctx.needs_input_grad[2], "CombinedRoPE does not support gradients in position embeddings"
        hs = ctx.heads_second
        doq, dok = _lastdim_contig(doq, dok)
        _seen(ctx.kernel_cache, "bwd", _sig(doq, dok, pos_emb) + (hs,))
        B, H, Tq, Tk, D = ctx.dims
        pe = _pos_emb_args(pos_emb, Tq, Tk)
        cq, ck = ctx.seq_cutoff
        dq, dk = torch.empty_like(doq), torch.empty_like(dok)
        lib = _hip.lib()
        _hip.check(lib.rgd_rope_qk(B, H, Tq, Tk, D, t4(doq, hs), t4(dok, hs), t4(dq, hs), t4(dk, hs), *pe, cq, ck, 1,
                                   _hip.dtype_code(doq.dtype), _hip.stream_ptr(doq.device)), "rgd_rope_qk")
        return dq, dk, None, None, None, None, None


def triton_rope_fn(query, key, pos_emb, seq_cutoff=None, heads_second=True, fused_ln=False, kernel_cache=None,
                   in_place=False):
    """Out of place unless in_place=True.  (The reference passes kernel_cache into the in_place slot,
    head_rope_cached.py:326-327, so its Module rotated q and k in place and never cached; `fused_ln`
    is ignored there as here.)"""
    return CombinedRoPEFunc.apply(query, key, pos_emb, seq_cutoff, heads_second, in_place, kernel_cache)


class FusedRoPEFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, pos_emb, seq_cutoff=None, heads_second=True, norm_eps=1e-6, kernel_cache=None):
        q, k, pos_emb = _lastdim_contig(q, k, _table_for(pos_emb, q))
        _seen(kernel_cache, "fwd", _sig(q, k, pos_emb) + (heads_second,))
        B, H, Tq, Tk, D = _qk_dims(q, k, heads_second, 128, "LayerNorm+RoPE")
        pe = _pos_emb_args(pos_emb, Tq, Tk)
        cq, ck = _cutoffs(seq_cutoff, Tq, Tk)
        qo, ko = torch.empty_like(q), torch.empty_like(k)
        lib = _hip.lib()
        _hip.check(lib.rgd_ln_rope_qk_fwd(B, H, Tq, Tk, D, t4(q, heads_second), t4(k, heads_second),
                                          t4(qo, heads_second), t4(ko, heads_second), *pe, cq, ck,
                                          _hip.dtype_code(q.dtype), float(norm_eps), _hip.stream_ptr(q.device)),
                   "rgd_ln_rope_qk_fwd")
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(q, k, pos_emb)
        ctx.seq_cutoff = (cq, ck)
        ctx.heads_second = heads_second
        ctx.norm_eps = float(norm_eps)
        ctx.dims = (B, H, Tq, Tk, D)
        return qo, ko

    @staticmethod
    def backward(ctx, doq, dok):
        _no_capture("FusedRoPEFunc.backward")
        q, k, pos_emb = ctx.saved_tensors
        assert not ctx.needs_input_grad[2], "CombinedRoPE does not support gradients in position embeddings"
        hs = ctx.heads_second
        doq, dok = _lastdim_contig(doq, dok)
        _seen(ctx.kernel_cache, "bwd", _sig(q, k, doq, dok, pos_emb) + (hs,))
        B, H, Tq, Tk, D = ctx.dims
        pe = _pos_emb_args(pos_emb, Tq, Tk)
        cq, ck = ctx.seq_cutoff
        dq, dk = torch.empty_like(q), torch.empty_like(k)
        lib = _hip.lib()
        _hip.check(lib.rgd_ln_rope_qk_bwd(B, H, Tq, Tk, D, t4(q, hs), t4(k, hs), t4(doq, hs), t4(dok, hs), t4(dq, hs),
                                          t4(dk, hs), *pe, cq, ck, _hip.dtype_code(q.dtype), ctx.norm_eps,
                                          _hip.stream_ptr(q.device)), "rgd_ln_rope_qk_bwd")
        return dq, dk, None, None, None, None, None


def triton_fused_ln_rope_fn(query, key, pos_emb, seq_cutoff=None, heads_second=True, norm_eps=1e-6, kernel_cache=None):
    return FusedRoPEFunc.apply(query, key, pos_emb, seq_cutoff, heads_second, norm_eps, kernel_cache)


# ----------------------------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------------------------


def _bias_args(bias, q, seqlen_q, seqlen_k, batch, nheads):
    """Bias classification of the reference (flash_attn_triton_cached.py:771-788): 4-D, dtype of q or
    fp32, last two dims (1, Tk) = "vector" or (Tq, Tk) = "matrix", leading dims broadcast."""
    if bias is None:
        return _hip.Tensor4(None, 0, 0, 0), _hip.BIAS_NONE, _hip.RGD_F32
    assert bias.dtype in [q.dtype, torch.float]
    assert bias.is_cuda
    assert bias.dim() == 4
    assert bias.stride(-1) == 1
    if bias.shape[2:] == (1, seqlen_k):
        kind = _hip.BIAS_VECTOR
    elif bias.shape[2:] == (seqlen_q, seqlen_k):
        kind = _hip.BIAS_MATRIX
    else:
        raise RuntimeError("Last 2 dimensions of bias must be (1, seqlen_k)" " or (seqlen_q, seqlen_k)")
    bias = bias.expand(batch, nheads, seqlen_q, seqlen_k)
    desc = _hip.Tensor4(bias.data_ptr(), bias.stride(0), bias.stride(1), bias.stride(2))
    return desc, kind, _hip.dtype_code(bias.dtype)


# The classes of the last head-shared bias seen on each device.  The layers of a model usually share one mask: the first
# attention call of a step classifies it, the others find the classes here.  An entry names the bias by its storage,
# view and version counter (in-place writes through any view bump it) and holds the storage, so that its address cannot
# be given to another tensor while the entry lives; one entry per device, replaced by the next bias.
# Writes that bypass the counter (through `.data`, or by a kernel that was handed the raw pointer) are not seen: call
# clear_bias_classes_cache() after them, or set RGD_CLASSES_CACHE=0.
_classes_cache = {}
_classes_cache_on = os.environ.get("RGD_CLASSES_CACHE", "1") != "0"


def clear_bias_classes_cache():
    """Forgets the tile classes kept for the last head-shared attention bias of every device."""
    _classes_cache.clear()


def _bias_classes(bias, bdesc, bkind, bdtype, dims):
    """Tile classes of a bias matrix that the heads share (rgd_attn_bias_classify): one pass over the bias, made in the
    forward and kept for the backward.  None when the library has no use for them (any other bias, head dims above 64)."""
    if bias is None:
        return None
    lib = _hip.lib()
    nbytes = lib.rgd_attn_bias_classes_bytes(*dims, bdesc, bkind, bdtype)
    if nbytes == 0:
        return None
    # under stream capture the classification must be part of the graph (a replay may find new values in the bias)
    cacheable = _classes_cache_on and not torch.cuda.is_current_stream_capturing()
    storage = bias.untyped_storage()
    # (the stream too: the classes are ready for work queued behind them on the stream that wrote them)
    key = (storage.data_ptr(), bias.storage_offset(), tuple(bias.shape), tuple(bias.stride()), bias.dtype, bias._version, dims,
           torch.cuda.current_stream(bias.device).cuda_stream)
    if cacheable:
        hit = _classes_cache.get(bias.device)
        if hit is not None and hit[0] == key:
            return hit[2]
    classes = torch.empty(nbytes // 8, dtype=torch.int64, device=bias.device)
    _hip.check(lib.rgd_attn_bias_classify(*dims, bdesc, bkind, bdtype, classes.data_ptr(), nbytes, _hip.stream_ptr(bias.device)),
               "rgd_attn_bias_classify")
    if cacheable:
        _classes_cache[bias.device] = (key, storage, classes)
    return classes


def _flash_attn_forward(q, k, v, bias=None, causal=False, softmax_scale=None, kernel_cache=None, return_classes=False):
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, _, _ = k.shape
    if not _seen(kernel_cache, "fwd", _sig(q, k, v, bias) + (bool(causal),)):
        assert k.shape == (batch, seqlen_k, nheads, d)
        assert v.shape == (batch, seqlen_k, nheads, d)
        assert d <= 128, "FlashAttention only support head dimensions up to 128"
        assert q.dtype == k.dtype == v.dtype, f"All tensors must have the same type {q.dtype=}, {k.dtype=}, {v.dtype=}"
        assert q.dtype in [torch.float16, torch.bfloat16], "Only support fp16 and bf16"
        assert q.is_cuda and k.is_cuda and v.is_cuda
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)
    if bias is not None and bias.stride(-1) != 1:
        bias = bias.contiguous()
    bdesc, bkind, bdtype = _bias_args(bias, q, seqlen_q, seqlen_k, batch, nheads)
    lib = _hip.lib()
    seqlen_q_rounded = lib.rgd_attn_seqlen_q_rounded(seqlen_q)
    lse = torch.empty((batch, nheads, seqlen_q_rounded), device=q.device, dtype=torch.float32)
    o = torch.empty_like(q)
    ws = _hip.workspace(q.device, lib.rgd_attn_fwd_workspace(batch, nheads, seqlen_q, seqlen_k, d))
    classes = _bias_classes(bias, bdesc, bkind, bdtype, (batch, nheads, seqlen_q, seqlen_k, d))
    _hip.check(lib.rgd_attn_fwd(batch, nheads, seqlen_q, seqlen_k, d, t4(q, False), t4(k, False), t4(v, False),
                                bdesc, bkind, bdtype, t4(o, False), ctypes.c_void_p(lse.data_ptr()),
                                _hip.dtype_code(q.dtype), int(bool(causal)), float(softmax_scale),
                                classes.data_ptr() if classes is not None else None,
                                ctypes.c_void_p(ws.data_ptr()), ws.numel(), _hip.stream_ptr(q.device)), "rgd_attn_fwd")
    if return_classes:
        return o, lse, softmax_scale, classes
    return o, lse, softmax_scale


_ATTN_BWD_MODES = {"auto": _hip.ATTN_BWD_AUTO, "two_kernel": _hip.ATTN_BWD_TWO_KERNEL, "one_pass": _hip.ATTN_BWD_ONE_PASS}
_attn_bwd_mode = os.environ.get("RGD_ATTN_BWD", "auto")
assert _attn_bwd_mode in _ATTN_BWD_MODES, f"RGD_ATTN_BWD must be one of {sorted(_ATTN_BWD_MODES)}"


def set_attention_backward(mode):
    """Form of the attention backward: "two_kernel" (every gradient reproducible bit for bit), "one_pass" (head dims up
    to 64: one kernel, dQ accumulated with fp32 atomics, so its last bits differ from run to run; dK and dV do not;
    wider heads run the two-kernel form) or "auto" (the library's choice).  `torch.use_deterministic_algorithms(True)`
    overrides it with "two_kernel".  Returns the previous setting."""
    global _attn_bwd_mode
    assert mode in _ATTN_BWD_MODES, f"mode must be one of {sorted(_ATTN_BWD_MODES)}"
    prev, _attn_bwd_mode = _attn_bwd_mode, mode
    return prev


def _bwd_mode(d):
    if torch.are_deterministic_algorithms_enabled():
        return _hip.ATTN_BWD_TWO_KERNEL
    if _attn_bwd_mode == "one_pass" and d > 64:
        return _hip.ATTN_BWD_TWO_KERNEL
    return _ATTN_BWD_MODES[_attn_bwd_mode]


# bytes of the buffer that receives dS of every (query, key) pair when a bias gradient is asked for; a bias that
# broadcasts over heads (or the batch) is served in chunks of heads (or batch elements) that fit it
_DBIAS_CHUNK_BYTES = int(os.environ.get("RGD_DBIAS_CHUNK_MB", "256")) << 20


def _attn_bwd_call(do, q, k, v, o, lse, dq, dk, dv, bias, causal, softmax_scale, mode, dfull, bias_classes):
    """One rgd_attn_bwd launch sequence on (B, T, H, D) tensors or views of them; lse is contiguous (B, H, Tq_rounded)."""
    batch, seqlen_q, nheads, d = q.shape
    seqlen_k = k.shape[1]
    lib = _hip.lib()
    bdesc, bkind, bdtype = _bias_args(bias, q, seqlen_q, seqlen_k, batch, nheads)
    ddesc = None
    if dfull is not None:
        ddesc = _hip.Tensor4(dfull.data_ptr(), dfull.stride(0), dfull.stride(1), dfull.stride(2))
    nbytes = lib.rgd_attn_bwd_workspace(batch, nheads, seqlen_q, seqlen_k, d, mode)
    ws = _hip.workspace(q.device, nbytes)
    _hip.check(lib.rgd_attn_bwd(batch, nheads, seqlen_q, seqlen_k, d, t4(do, False), t4(q, False), t4(k, False),
                                t4(v, False), t4(o, False), ctypes.c_void_p(lse.data_ptr()), bdesc, bkind, bdtype,
                                t4(dq, False), t4(dk, False), t4(dv, False), ddesc, _hip.dtype_code(q.dtype),
                                int(bool(causal)), float(softmax_scale), mode,
                                bias_classes.data_ptr() if bias_classes is not None else None, ws.data_ptr(), nbytes,
                                _hip.stream_ptr(q.device)), "rgd_attn_bwd")


def _flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, bias=None, causal=False, softmax_scale=None,
                         kernel_cache=None, bias_grad=False, bias_classes=None):
    """Returns None, or with bias_grad the gradient of `bias` in its own shape and dtype (beyond the reference, which
    refuses it, flash_attn_triton_cached.py:1107): the dQ kernel leaves dS of every (query, key) pair, rounded to the
    bias dtype, in a (B, H, Tq, Tk) buffer and the dimensions the bias broadcasts are summed here in fp32.  A bias
    that broadcasts over the heads (else: over the batch) is served in chunks of heads (batch elements), so that the
    buffer stays within RGD_DBIAS_CHUNK_MB (256) MiB where one head (batch element) fits that."""
    if do.stride(-1) != 1:
        do = do.contiguous()
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, _, _ = k.shape
    lib = _hip.lib()
    seqlen_q_rounded = lib.rgd_attn_seqlen_q_rounded(seqlen_q)
    if not _seen(kernel_cache, "bwd", _sig(q, k, v, bias, do) + (bool(causal),)):
        assert d <= 128
        assert lse.shape == (batch, nheads, seqlen_q_rounded)
        assert q.stride(-1) == k.stride(-1) == v.stride(-1) == o.stride(-1) == 1
        assert dq.stride(-1) == dk.stride(-1) == dv.stride(-1) == 1
    _seen(kernel_cache, "bwd_odot", _sig(o, do))
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)
    if not bias_grad:
        _attn_bwd_call(do, q, k, v, o, lse, dq, dk, dv, bias, causal, softmax_scale, _bwd_mode(d), None, bias_classes)
        return None

    mode = _hip.ATTN_BWD_TWO_KERNEL  # the dQ kernel writes the bias gradient
    tk_pad = (seqlen_k + 63) // 64 * 64  # rows of whole 64-key tiles
    alloc = torch.zeros if causal else torch.empty  # key tiles past the causal diagonal are not visited
    over_heads = bias.shape[1] == 1 and nheads > 1
    over_batch = bias.shape[0] == 1 and batch > 1
    pair_bytes = seqlen_q * tk_pad * bias.element_size()
    hc, bc = nheads, batch
    if over_heads:
        hc = max(1, min(nheads, _DBIAS_CHUNK_BYTES // max(1, batch * pair_bytes)))
    elif over_batch:
        bc = max(1, min(batch, _DBIAS_CHUNK_BYTES // max(1, nheads * pair_bytes)))
    if hc == nheads and bc == batch:
        dfull = alloc((batch, nheads, seqlen_q, tk_pad), dtype=bias.dtype, device=q.device)
        _attn_bwd_call(do, q, k, v, o, lse, dq, dk, dv, bias, causal, softmax_scale, mode, dfull, None)
        dfull = dfull[..., :seqlen_k]
        dims = [i for i in range(4) if bias.shape[i] == 1 and dfull.shape[i] != 1]
        if dims:
            return dfull.sum(dim=dims, keepdim=True, dtype=torch.float32).to(bias.dtype)
        return dfull.contiguous()

    acc = torch.zeros(bias.shape, dtype=torch.float32, device=q.device)
    buf = alloc((bc, hc, seqlen_q, tk_pad), dtype=bias.dtype, device=q.device)
    for b0 in range(0, batch, bc):
        for h0 in range(0, nheads, hc):
            bs, hs = slice(b0, min(batch, b0 + bc)), slice(h0, min(nheads, h0 + hc))
            part = buf[: bs.stop - bs.start, : hs.stop - hs.start]
            if causal and (b0 or h0):
                part.zero_()
            bias_part = bias[bs if bias.shape[0] > 1 else slice(None), hs if bias.shape[1] > 1 else slice(None)]
            _attn_bwd_call(do[bs, :, hs], q[bs, :, hs], k[bs, :, hs], v[bs, :, hs], o[bs, :, hs], lse[bs, hs].contiguous(),
                           dq[bs, :, hs], dk[bs, :, hs], dv[bs, :, hs], bias_part, causal, softmax_scale, mode, part, None)
            got = part[..., :seqlen_k]
            dims = [i for i in range(4) if bias.shape[i] == 1 and got.shape[i] != 1]
            got = got.sum(dim=dims, keepdim=True, dtype=torch.float32) if dims else got.float()
            acc[bs if bias.shape[0] > 1 else slice(None), hs if bias.shape[1] > 1 else slice(None)] += got
    return acc.to(bias.dtype)


class FlashAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, bias=None, causal=False, softmax_scale=None, kernel_cache=None):
        """
        q: (batch_size, seqlen_q, nheads, headdim)
        k, v: (batch_size, seqlen_k, nheads, headdim)
        bias: optional, shape broadcastible to (batch, nheads, seqlen_q, seqlen_k).
        """
        q, k, v, bias = _lastdim_contig(q, k, v, bias)
        o, lse, ctx.softmax_scale, ctx.bias_classes = _flash_attn_forward(
            q, k, v, bias=bias, causal=causal, softmax_scale=softmax_scale, kernel_cache=kernel_cache, return_classes=True)
        ctx.kernel_cache = kernel_cache
        ctx.save_for_backward(q, k, v, o, lse, bias)
        ctx.causal = causal
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, dlse):
        _no_capture("FlashAttnFunc.backward")
        q, k, v, o, lse, bias = ctx.saved_tensors
        # the reference stops here with "FlashAttention does not support bias gradient yet"
        # (flash_attn_triton_cached.py:1107); this implementation provides it
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dbias = _flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, bias=bias, causal=ctx.causal,
                                     softmax_scale=ctx.softmax_scale, kernel_cache=ctx.kernel_cache,
                                     bias_grad=bias is not None and ctx.needs_input_grad[3], bias_classes=ctx.bias_classes)
        return dq, dk, dv, dbias, None, None, None


def flash_attn_func(q, k, v, bias=None, causal=False, softmax_scale=None, return_lse=False, kernel_cache=None):
    o, lse = FlashAttnFunc.apply(q, k, v, bias, causal, softmax_scale, kernel_cache)
    return (o, lse) if return_lse else o
