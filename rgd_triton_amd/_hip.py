"""ctypes binding of librgd_hip.so (declared in include/rgd_hip.h).

The library is built in-tree by `make -C rgd_triton_amd/csrc` (or `__graft_entry__.build()`).
There is no fallback path: if the library is missing, every operator raises.
"""
import ctypes
import os
import re
import threading
import warnings

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# RGD_HIP_LIB overrides the library path (used to compare kernel build variants)
LIB_PATH = os.environ.get("RGD_HIP_LIB") or os.path.join(_HERE, "librgd_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "rgd_hip.h")

RGD_F32, RGD_F16, RGD_BF16 = 0, 1, 2
ABI_MAJOR = 3  # rgd_version() // 1000 this binding was written for
BIAS_NONE, BIAS_VECTOR, BIAS_MATRIX = 0, 1, 2
ATTN_BWD_AUTO, ATTN_BWD_TWO_KERNEL, ATTN_BWD_ONE_PASS = 0, 1, 2

_DTYPE_CODE = {torch.float32: RGD_F32, torch.float16: RGD_F16, torch.bfloat16: RGD_BF16}


class Tensor3(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_n", ctypes.c_int64)]


class Tensor4(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64),
                ("stride_n", ctypes.c_int64)]


_i64, _int, _f32, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
_T3, _T4 = ctypes.POINTER(Tensor3), ctypes.POINTER(Tensor4)

# argument types of every entry point, in the order of include/rgd_hip.h
_SIGNATURES = {
    "rgd_version": (_int, []),
    "rgd_last_error": (ctypes.c_char_p, []),
    "rgd_init": (_int, []),
    "rgd_rms_fwd": (_int, [_i64, _i64, _i64, _T3, _T3, _T3, _int, _int, _f32, _vp]),
    "rgd_rms_bwd_workspace": (_sz, [_i64] * 5),
    "rgd_rms_bwd": (_int, [_i64, _i64, _i64, _T3, _T3, _T3, _T3, _T3, _int, _int, _int, _f32, _vp, _sz, _vp]),
    "rgd_rms_bwd_noalloc_limit": (_sz, []),
    "rgd_rms_bwd_noalloc": (_int, [_i64, _i64, _i64, _T3, _T3, _T3, _T3, _T3, _int, _int, _int, _f32, _vp]),
    "rgd_fused_rms_fwd": (_int, [_i64] * 5 + [_T3] * 6 + [_int, _int, _int, _f32, _vp]),
    "rgd_fused_rms_bwd": (_int, [_i64] * 5 + [_T3] * 5 + [_int] + [_T3] * 5 + [_int] + [_int, _int, _int, _f32,
                                                                                 _vp, _sz, _vp]),
    "rgd_l2_fwd": (_int, [_i64, _i64, _i64, _T3, _T3, _int, _f32, _vp]),
    "rgd_l2_bwd": (_int, [_i64, _i64, _i64, _T3, _T3, _T3, _int, _f32, _vp]),
    "rgd_fused_l2_fwd": (_int, [_i64] * 5 + [_T3] * 4 + [_int, _f32, _vp]),
    "rgd_fused_l2_bwd": (_int, [_i64] * 5 + [_T3] * 6 + [_int, _f32, _vp]),
    "rgd_ln_qk_fwd": (_int, [_i64] * 5 + [_T4] * 4 + [_int, _f32, _vp]),
    "rgd_ln_qk_bwd": (_int, [_i64] * 5 + [_T4] * 6 + [_int, _f32, _vp]),
    "rgd_rope_qk": (_int, [_i64] * 5 + [_T4] * 4 + [_vp, _i64, _i64, _i64, _i64, _int, _i64, _i64, _int, _int, _vp]),
    "rgd_ln_rope_qk_fwd": (_int, [_i64] * 5 + [_T4] * 4 + [_vp, _i64, _i64, _i64, _i64, _int, _i64, _i64, _int, _f32,
                                                            _vp]),
    "rgd_ln_rope_qk_bwd": (_int, [_i64] * 5 + [_T4] * 6 + [_vp, _i64, _i64, _i64, _i64, _int, _i64, _i64, _int, _f32,
                                                            _vp]),
    "rgd_attn_seqlen_q_rounded": (_i64, [_i64]),
    "rgd_attn_bias_classes_bytes": (_sz, [_i64] * 5 + [_T4, _int, _int]),
    "rgd_attn_bias_classify": (_int, [_i64] * 5 + [_T4, _int, _int, _vp, _sz, _vp]),
    "rgd_attn_fwd": (_int, [_i64] * 5 + [_T4] * 4 + [_int, _int, _T4, _vp, _int, _int, _f32, _vp, _vp, _sz, _vp]),
    "rgd_attn_fwd_workspace": (_sz, [_i64] * 5),
    "rgd_attn_bwd_workspace": (_sz, [_i64] * 5 + [_int]),
    "rgd_attn_bwd": (_int, [_i64] * 5 + [_T4] * 5 + [_vp] + [_T4, _int, _int] + [_T4] * 4 + [_int, _int, _f32, _int, _vp,
                                                                                         _vp, _sz, _vp]),
}

_lib = None
_lock = threading.Lock()


def declared_symbols(header_path=HEADER_PATH):
    """Names of every function include/rgd_hip.h declares."""
    text = open(header_path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rgd_[a-z0-9_]+)\s*\(", text)))


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')} -j8` "
                    "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no fallback path.")
            handle = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(handle, name)  # AttributeError if the library does not export it
                fn.restype = res
                fn.argtypes = args
            if handle.rgd_version() // 1000 != ABI_MAJOR:
                raise RuntimeError(f"{LIB_PATH} has ABI version {handle.rgd_version()}, this package needs "
                                   f"{ABI_MAJOR}xxx: rebuild it")
            # one-time set-up now (kernel attributes, device properties), so that no entry point has any left to
            # do when it first runs, e.g. under stream capture.  Without a GPU the call only records that.
            if torch.cuda.is_available():
                rc = handle.rgd_init()
                if rc != 0:
                    # what failed is reported again, as an error, by the entry points that need it (the attention
                    # kernels' set-up); the row kernels need none of it and stay usable
                    warnings.warn(f"rgd_init failed ({rc}): {handle.rgd_last_error().decode(errors='replace')}",
                                  RuntimeWarning)
            _lib = handle
    return _lib


def check(rc, what):
    if rc != 0:
        msg = lib().rgd_last_error().decode(errors="replace")
        raise RuntimeError(f"{what} failed ({rc}): {msg}")


def dtype_code(dtype, msg="Only support fp16, bf16, and fp32"):
    assert dtype in _DTYPE_CODE, msg
    return _DTYPE_CODE[dtype]


def t3(t, stride_b=None):
    """(B,T,C) tensor -> Tensor3; a 1-row weight passes stride_b explicitly."""
    return Tensor3(t.data_ptr(), t.stride(0) if stride_b is None else stride_b, t.stride(1) if t.dim() > 1 else 0)


def t4(t, heads_second):
    """(B,H,T,D) or (B,T,H,D) tensor -> Tensor4 with (batch, head, token) strides."""
    if heads_second:
        return Tensor4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
    return Tensor4(t.data_ptr(), t.stride(0), t.stride(2), t.stride(1))


def stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def workspace(device, nbytes):
    """Scratch for ONE call: a fresh uint8 tensor from PyTorch's caching allocator.  The allocator hands a freed
    block only to later work of the same stream, so the buffer is safe to drop as soon as the call has been
    enqueued, calls on different streams or host threads never share one, and under graph capture the block
    comes from the graph's private pool (the reference allocates delta and dq_accum per call in the same way,
    flash_attn/flash_attn_triton_cached.py:896-900)."""
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)
