"""Seeded random shapes, layouts, strides and options for every operator, against the CPU oracle.
The fixed parametrisations of the other test files follow the reference's tests; this file walks the
space between them (odd lengths around the tile sizes, unaligned views, every bias form, causal, scale,
cutoffs) with cases small enough for the oracle to finish in milliseconds."""
import math
import random

import pytest
import torch

from helpers import assert_close, assert_close_allow_inf, dev, gen, oracle, randn, to_gpu
from test_flash_attn import check, reference

pytestmark = pytest.mark.gpu

DT3 = [torch.float32, torch.float16, torch.bfloat16]
DT2 = [torch.float16, torch.bfloat16]


def _lengths(rng):
    """a length near a tile boundary more often than not"""
    base = rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 191, 192, 200, 255, 256, 257, 300, 383, 385, 512, 640])
    return max(1, base + rng.choice([0, 0, 0, -1, 1, 7]))


def _strided(g, rng, shape, dtype, scale=1.0, shift=0.0):
    """a tensor of `shape` that is a view into a larger buffer about one time in three"""
    kind = rng.choice(["plain", "plain", "pad_last", "pad_tokens"])
    if kind == "plain":
        return randn(g, *shape, dtype=dtype, scale=scale, shift=shift)
    if kind == "pad_last":  # rows inside a wider buffer (row stride != D, possibly unaligned)
        pad = rng.choice([1, 3, 8, 16])
        big = randn(g, *shape[:-1], shape[-1] + pad, dtype=dtype, scale=scale, shift=shift)
        off = rng.choice([0, pad])
        return big[..., off:off + shape[-1]]
    big = randn(g, shape[0], shape[1] + 3, *shape[2:], dtype=dtype, scale=scale, shift=shift)
    return big[:, 2:2 + shape[1]]


@pytest.mark.parametrize("seed", range(120))
def test_random_attention(seed):
    from rgd_triton_amd import flash_attn_func

    rng = random.Random(1000 + seed)
    g = gen(2000 + seed)
    dtype = rng.choice(DT2)
    B, H = rng.choice([(1, 1), (2, 3), (3, 2), (1, 5)])
    Tq, Tk = _lengths(rng), _lengths(rng)
    d = rng.choice([8, 16, 24, 32, 40, 59, 64, 72, 96, 111, 128])
    causal = rng.random() < 0.25
    kind = rng.choice(["none", "none", "static", "batch", "head", "cube", "vector"])
    bias_dtype = rng.choice([dtype, dtype, torch.float32])
    q = _strided(g, rng, (B, Tq, H, d), dtype)
    k = _strided(g, rng, (B, Tk, H, d), dtype)
    v = _strided(g, rng, (B, Tk, H, d), dtype)
    do = _strided(g, rng, (B, Tq, H, d), dtype)
    shape = {"none": None, "static": (1, 1, Tq, Tk), "batch": (B, 1, Tq, Tk), "head": (1, H, Tq, Tk),
             "cube": (B, H, Tq, Tk), "vector": (B, H, 1, Tk)}[kind]
    bias = None if shape is None else randn(g, *shape, dtype=bias_dtype)
    if bias is not None and rng.random() < 0.4:  # mask some keys for everybody, never all of them
        dead = torch.randperm(Tk, generator=g)[: Tk // 3]
        dead = dead[dead != 0]  # with a causal mask the first query row sees key 0 only: keep it, so that no row
        bias[..., dead] = float("-inf")  # is fully masked (the PyTorch reference gives NaN there, the kernels 0)
    qg, kg, vg = to_gpu(q, k, v, requires_grad=True)
    o, lse = flash_attn_func(qg, kg, vg, None if bias is None else bias.to("cuda"), causal, None, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), dev(do))
    ref = reference(q, k, v, bias, do, causal)
    if bias is not None and bias.dtype != dtype:  # the low-precision comparison run adds the bias in q's dtype
        ref = ref[:3] + reference(q, k, v, bias.to(dtype), do, causal)[3:]
    check((o, lse, dq, dk, dv), ref, Tq, grad_mult=3, grad_add=2e-3,
          name=f"seed {seed}: {dtype} B{B} H{H} Tq{Tq} Tk{Tk} d{d} causal={causal} bias={kind}/{bias_dtype}")


@pytest.mark.parametrize("seed", range(100))
def test_random_wide_rows(seed):
    from rgd_triton_amd import (triton_fused_norm_func_fn, triton_fused_rms_func_fn, triton_norm_func_fn,
                                triton_rms_func_fn)

    rng = random.Random(3000 + seed)
    g = gen(4000 + seed)
    dtype = rng.choice(DT3)
    B = rng.choice([1, 2, 5])
    T1, T2 = _lengths(rng), _lengths(rng)
    C1 = rng.choice([8, 24, 33, 64, 100, 256, 384, 513, 768, 1000, 1024, 1536, 2047, 2048, 2560, 3072, 4096, 5000, 8192])
    C2 = rng.choice([16, 97, 256, 1024, 1536])
    op = rng.choice(["rms", "rms2", "l2", "l2x2"])
    x1, d1 = _strided(g, rng, (B, T1, C1), dtype), _strided(g, rng, (B, T1, C1), dtype)
    x2, d2 = _strided(g, rng, (B, T2, C2), dtype), _strided(g, rng, (B, T2, C2), dtype)
    name = f"seed {seed}: {op} {dtype} B{B} T{T1},{T2} C{C1},{C2}"
    if op in ("rms", "rms2"):
        unique = rng.random() < 0.5
        wdtype = rng.choice([dtype, dtype, torch.float32])
        w1 = (1 + 0.1 * torch.randn((B, 1, C1) if unique else (C1,), generator=g)).to(wdtype)
        w2 = (1 + 0.1 * torch.randn((B, 1, C2) if unique else (C2,), generator=g)).to(wdtype)
        rows1, rows2 = (T1 if unique else B * T1), (T2 if unique else B * T2)
        if op == "rms":
            xg, wg = to_gpu(x1, w1, requires_grad=True)
            y = triton_rms_func_fn(xg, wg, 1e-6)
            dx, dw = torch.autograd.grad(y, (xg, wg), dev(d1))
            dx_r, dw_r = oracle.rms_bwd(d1, x1, w1, 1e-6)
            assert_close(y, oracle.rms_fwd(x1, w1, 1e-6), dtype, "rms", name + " y")
            assert_close(dx, dx_r, dtype, "rms", name + " dx")
            assert_close(dw, dw_r, wdtype, "rms", name + " dw", atol_scale=3 * rows1 * C1 ** 0.5)
        else:
            a, b_, wa, wb = to_gpu(x1, x2, w1, w2, requires_grad=True)
            y1, y2 = triton_fused_rms_func_fn(a, b_, wa, wb, 1e-6)
            ga = torch.autograd.grad((y1, y2), (a, b_, wa, wb), (dev(d1), dev(d2)))
            r1, r2 = oracle.rms_bwd(d1, x1, w1, 1e-6), oracle.rms_bwd(d2, x2, w2, 1e-6)
            assert_close(y1, oracle.rms_fwd(x1, w1, 1e-6), dtype, "rms", name + " y1")
            assert_close(y2, oracle.rms_fwd(x2, w2, 1e-6), dtype, "rms", name + " y2")
            assert_close(ga[0], r1[0], dtype, "rms", name + " dx1")
            assert_close(ga[1], r2[0], dtype, "rms", name + " dx2")
            assert_close(ga[2], r1[1], wdtype, "rms", name + " dw1", atol_scale=3 * rows1 * C1 ** 0.5)
            assert_close(ga[3], r2[1], wdtype, "rms", name + " dw2", atol_scale=3 * rows2 * C2 ** 0.5)
    elif op == "l2":
        xg = to_gpu(x1, requires_grad=True)
        y = triton_norm_func_fn(xg, 1e-6)
        (dx,) = torch.autograd.grad(y, xg, dev(d1))
        assert_close(y, oracle.l2_fwd(x1, 1e-6), dtype, name=name + " y")
        assert_close_allow_inf(dx, oracle.l2_bwd(d1, x1, 1e-6), dtype, name=name + " dx")
    else:
        a, b_ = to_gpu(x1, x2, requires_grad=True)
        y1, y2 = triton_fused_norm_func_fn(a, b_, 1e-6)
        ga = torch.autograd.grad((y1, y2), (a, b_), (dev(d1), dev(d2)))
        assert_close(y1, oracle.l2_fwd(x1, 1e-6), dtype, name=name + " y1")
        assert_close(y2, oracle.l2_fwd(x2, 1e-6), dtype, name=name + " y2")
        assert_close_allow_inf(ga[0], oracle.l2_bwd(d1, x1, 1e-6), dtype, name=name + " dx1")
        assert_close_allow_inf(ga[1], oracle.l2_bwd(d2, x2, 1e-6), dtype, name=name + " dx2")


@pytest.mark.parametrize("seed", range(100))
def test_random_head_ops(seed):
    from rgd_triton_amd import triton_fused_ln_func_fn, triton_fused_ln_rope_fn, triton_rope_fn

    rng = random.Random(5000 + seed)
    g = gen(6000 + seed)
    dtype = rng.choice(DT3)
    B, H = rng.choice([(1, 1), (2, 3), (3, 5)])
    Tq, Tk = _lengths(rng), _lengths(rng)
    op = rng.choice(["ln", "rope", "ln_rope"])
    heads_second = rng.random() < 0.5
    D = rng.choice([32, 40, 59, 64, 96, 128, 200, 256]) if op == "ln" else rng.choice([32, 48, 64, 96, 128])
    shape = (lambda T: (B, H, T, D)) if heads_second else (lambda T: (B, T, H, D))
    q, k = _strided(g, rng, shape(Tq), dtype, 1.5, 0.3), _strided(g, rng, shape(Tk), dtype, 1.5, 0.3)
    gq, gk = _strided(g, rng, shape(Tq), dtype), _strided(g, rng, shape(Tk), dtype)
    name = f"seed {seed}: {op} {dtype} B{B} H{H} Tq{Tq} Tk{Tk} D{D} heads_second={heads_second}"
    qg, kg = to_gpu(q, k, requires_grad=True)
    if op == "ln":
        qo, ko = triton_fused_ln_func_fn(qg, kg, heads_second, 1e-6)
        dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (dev(gq), dev(gk)))
        for a, r, n in ((qo, oracle.head_ln_fwd(q), "qo"), (ko, oracle.head_ln_fwd(k), "ko"),
                        (dq, oracle.head_ln_bwd(gq, q), "dq"), (dk, oracle.head_ln_bwd(gk, k), "dk")):
            assert_close(a, r, dtype, name=f"{name} {n}")
        return
    R = rng.choice([r for r in (8, 16, 32, 48, 64, 96, 128) if r <= D])
    P = max(Tq, Tk) + 1 + rng.choice([0, 5])
    table_dtype = rng.choice([dtype, torch.float32])
    pe = oracle.rotary_table(P, R, 10000.0, table_dtype)
    cutoff = (rng.choice([0, Tq // 2, Tq]), rng.choice([0, Tk // 2, Tk]))
    if op == "rope":
        qo, ko = triton_rope_fn(qg, kg, pe.to("cuda"), seq_cutoff=cutoff, heads_second=heads_second)
        ref_f = oracle.rope_fwd(q, k, pe, cutoff, heads_second)
        ref_b = oracle.rope_bwd(gq, gk, pe, cutoff, heads_second)
        tol = "rope"
    else:
        qo, ko = triton_fused_ln_rope_fn(qg, kg, pe.to("cuda"), seq_cutoff=cutoff, heads_second=heads_second, norm_eps=1e-6)
        ref_f = oracle.ln_rope_fwd(q, k, pe, cutoff, heads_second, 1e-6)
        ref_b = oracle.ln_rope_bwd(gq, gk, q, k, pe, cutoff, heads_second, 1e-6)
        tol = "ln_rope"
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (dev(gq), dev(gk)))
    for a, r, n in ((qo, ref_f[0], "qo"), (ko, ref_f[1], "ko"), (dq, ref_b[0], "dq"), (dk, ref_b[1], "dk")):
        assert_close(a, r, dtype, tol, f"{name} {n}")
