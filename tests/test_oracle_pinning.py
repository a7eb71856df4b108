"""Pins the CPU oracle (oracle/rgd_oracle.py) WITHOUT the reference: every function is checked against
a library routine, a closed form, brute force on tiny inputs in fp64, or an invariant, chosen so that a
dropped term, a wrong sign or index, or a transposed operand fails.  Runs on the CPU.

The reference holds no golden vectors or fixtures for this path (its tests draw random inputs on the
GPU at run time), so the tolerance tables are the only thing taken from its tests; they are checked
at the end of this file."""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import gen, oracle, randn

F64 = torch.float64


def r64(g, *shape):
    return torch.randn(*shape, generator=g, dtype=F64)


# ------------------------------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("wshape", ["vec", "one", "batch"])
def test_rms_against_library_and_autograd(wshape):
    g = gen(0)
    B, T, C = 3, 5, 37
    x, dy = r64(g, B, T, C), r64(g, B, T, C)
    w = {"vec": r64(g, C), "one": r64(g, 1, 1, C), "batch": r64(g, B, 1, C)}[wshape]
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y_lib = F.rms_norm(xr, (C,), None, 1e-6) * wr
    dx_lib, dw_lib = torch.autograd.grad(y_lib, (xr, wr), dy)
    torch.testing.assert_close(oracle.rms_fwd(x, w, 1e-6, F64), y_lib.detach(), rtol=1e-12, atol=1e-12)
    dx, dw = oracle.rms_bwd(dy, x, w, 1e-6, F64)
    assert dw.shape == w.shape
    torch.testing.assert_close(dx, dx_lib, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dw, dw_lib, rtol=1e-10, atol=1e-12)


def test_rms_hand_loop():
    x = torch.tensor([[[3.0, 4.0], [1.0, -1.0]]], dtype=F64)
    w = torch.tensor([2.0, 0.5], dtype=F64)
    y = oracle.rms_fwd(x, w, 0.0, F64)
    # row (3,4): rms = sqrt(12.5); row (1,-1): rms = 1
    exp = torch.tensor([[[3 / math.sqrt(12.5) * 2, 4 / math.sqrt(12.5) * 0.5], [2.0, -0.5]]], dtype=F64)
    torch.testing.assert_close(y, exp, rtol=1e-14, atol=0)
    # eps enters under the square root, added to the mean square
    y_eps = oracle.rms_fwd(x, w, 3.5, F64)
    assert abs(y_eps[0, 0, 0].item() - 3 / 4.0 * 2) < 1e-14


# ------------------------------------------------------------------------------------------ L2
def test_l2_against_library_and_autograd():
    g = gen(1)
    x, dy = r64(g, 2, 6, 19) * 100, r64(g, 2, 6, 19)
    xr = x.clone().requires_grad_(True)
    y_lib = F.normalize(xr, p=2, eps=1e-6, dim=-1)
    (dx_lib,) = torch.autograd.grad(y_lib, xr, dy)
    torch.testing.assert_close(oracle.l2_fwd(x, 1e-6, F64), y_lib.detach(), rtol=1e-12, atol=1e-14)
    torch.testing.assert_close(oracle.l2_bwd(dy, x, 1e-6, F64), dx_lib, rtol=1e-9, atol=1e-14)


def test_l2_clamped_rows_closed_form():
    x = torch.tensor([[[3e-4, 4e-4], [0.0, 0.0], [3.0, 4.0]]], dtype=F64)  # lengths 5e-4, 0, 5
    eps = 1e-2
    y = oracle.l2_fwd(x, eps, F64)
    torch.testing.assert_close(y[0, 0], x[0, 0] / eps)
    assert torch.all(y[0, 1] == 0)
    torch.testing.assert_close(y[0, 2], torch.tensor([0.6, 0.8], dtype=F64))
    torch.testing.assert_close(y, F.normalize(x, p=2, eps=eps, dim=-1))
    # clamped rows use the same backward expression with rlen = 1/eps (the reference's choice)
    dy = torch.tensor([[[1.0, 2.0], [1.0, 1.0], [0.5, -1.0]]], dtype=F64)
    dx = oracle.l2_bwd(dy, x, eps, F64)
    xh = x[0, 0] / eps
    torch.testing.assert_close(dx[0, 0], (dy[0, 0] - xh * (xh * dy[0, 0]).sum()) / eps)
    torch.testing.assert_close(dx[0, 1], dy[0, 1] / eps)


# ------------------------------------------------------------------------------------------ head LN
@pytest.mark.parametrize("heads_second", [True, False])
def test_head_ln_against_library_and_autograd(heads_second):
    g = gen(2)
    shape = (2, 3, 7, 24) if heads_second else (2, 7, 3, 24)
    x, dy = r64(g, *shape) * 3 + 1, r64(g, *shape)
    xr = x.clone().requires_grad_(True)
    y_lib = F.layer_norm(xr, (24,), None, None, 1e-6)
    (dx_lib,) = torch.autograd.grad(y_lib, xr, dy)
    torch.testing.assert_close(oracle.head_ln_fwd(x, 1e-6, F64), y_lib.detach(), rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(oracle.head_ln_bwd(dy, x, 1e-6, F64), dx_lib, rtol=1e-9, atol=1e-12)
    # invariants: zero mean, unit (biased) variance, gradient orthogonal to constants
    y = oracle.head_ln_fwd(x, 0.0, F64)
    assert y.mean(-1).abs().max() < 1e-13 and (y.var(-1, unbiased=False) - 1).abs().max() < 1e-12
    assert oracle.head_ln_bwd(dy, x, 1e-6, F64).sum(-1).abs().max() < 1e-10


# ------------------------------------------------------------------------------------------ RoPE
def test_rotary_table_closed_form():
    pe = oracle.rotary_table(50, 8, 10000.0)
    assert pe.shape == (2, 50, 8)
    t, i = 17, 2
    ang = t * 10000.0 ** (-2 * i / 8)
    assert abs(pe[0, t, 2 * i].item() - math.sin(ang)) < 1e-5 and abs(pe[1, t, 2 * i + 1].item() - math.cos(ang)) < 1e-5
    assert torch.equal(pe[:, :, 0::2], pe[:, :, 1::2])  # pair duplication
    torch.testing.assert_close(pe[0] ** 2 + pe[1] ** 2, torch.ones(50, 8), rtol=0, atol=1e-6)
    ax = oracle.axial_rotary_table(6, 16, 32.0)
    assert ax.shape == (2, 36, 16) and torch.equal(ax[:, :, 0::2], ax[:, :, 1::2])
    # first half of the channels follows x (fast index), second half y (slow index)
    assert torch.equal(ax[:, 0:6, :8], ax[:, 6:12, :8]) and torch.equal(ax[:, 0, 8:], ax[:, 5, 8:])
    assert not torch.equal(ax[:, 0, 8:], ax[:, 6, 8:])


@pytest.mark.parametrize("heads_second", [True, False])
def test_rope_is_complex_rotation(heads_second):
    """(x0 + i x1) * exp(i angle) for tokens < cutoff and channels < R; identity elsewhere"""
    g = gen(3)
    B, H, T, D, R = 2, 3, 9, 12, 8
    shape = (B, H, T, D) if heads_second else (B, T, H, D)
    q, k = r64(g, *shape), r64(g, *shape)
    pe = oracle.rotary_table(T + 1, R).to(F64)
    cut = (5, 9)
    qo, ko = oracle.rope_fwd(q, k, pe, cut, heads_second, F64)
    rot = torch.complex(pe[1, :T, ::2], pe[0, :T, ::2])  # cos + i sin, (T, R/2)
    for x, xo, c in ((q, qo, 5), (k, ko, 9)):
        xs = x if heads_second else x.transpose(1, 2)
        os_ = xo if heads_second else xo.transpose(1, 2)
        z = torch.complex(xs[..., :R:2], xs[..., 1:R:2]) * rot[None, None]
        exp = xs.clone()
        exp[:, :, :c, 0:R:2] = z.real[:, :, :c]
        exp[:, :, :c, 1:R:2] = z.imag[:, :, :c]
        torch.testing.assert_close(os_, exp, rtol=1e-12, atol=1e-13)
    # norm preserving per pair, exact copy beyond the cutoff and beyond R
    # (the table is built in fp32, so sin^2 + cos^2 = 1 only to fp32 accuracy)
    torch.testing.assert_close(qo.pow(2).sum(-1), q.pow(2).sum(-1), rtol=1e-6, atol=1e-6)
    assert torch.equal(oracle.rope_fwd(q, k, pe, 0, heads_second, F64)[0], q)


def test_rope_backward_is_transpose_for_pair_duplicated_tables():
    g = gen(4)
    q, k = r64(g, 2, 3, 7, 16).requires_grad_(True), r64(g, 2, 3, 11, 16).requires_grad_(True)
    gq, gk = r64(g, 2, 3, 7, 16), r64(g, 2, 3, 11, 16)
    pe = oracle.rotary_table(12, 8).to(F64)
    qo, ko = oracle.rope_fwd(q, k, pe, (6, 11), True, F64)
    dq_ad, dk_ad = torch.autograd.grad((qo, ko), (q, k), (gq, gk))
    dq, dk = oracle.rope_bwd(gq, gk, pe, (6, 11), True, F64)
    torch.testing.assert_close(dq, dq_ad, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(dk, dk_ad, rtol=1e-12, atol=1e-13)
    # bwd(fwd(x)) == x because sin^2 + cos^2 == 1
    back, _ = oracle.rope_bwd(qo.detach(), ko.detach(), pe, (6, 11), True, F64)
    torch.testing.assert_close(back, q.detach(), rtol=1e-6, atol=1e-6)


def test_rope_backward_sign_convention_for_general_tables():
    """with a table that is NOT pair duplicated the reference's backward (sin/cos at the output channel,
    rotation sign flipped) differs from the transpose; the oracle must follow the reference"""
    x = torch.tensor([[[[1.0, 2.0]]]], dtype=F64)
    pe = torch.tensor([[[0.1, 0.3]], [[0.9, 0.7]]], dtype=F64).repeat(1, 2, 1)  # sin (0.1, 0.3), cos (0.9, 0.7)
    fo, _ = oracle.rope_fwd(x, x, pe, None, True, F64)
    torch.testing.assert_close(fo[0, 0, 0], torch.tensor([1 * 0.9 - 2 * 0.1, 2 * 0.7 + 1 * 0.3], dtype=F64))
    bo, _ = oracle.rope_bwd(x, x, pe, None, True, F64)
    torch.testing.assert_close(bo[0, 0, 0], torch.tensor([1 * 0.9 + 2 * 0.1, 2 * 0.7 - 1 * 0.3], dtype=F64))


@pytest.mark.parametrize("heads_second", [True, False])
def test_ln_rope_is_composition_and_matches_autograd(heads_second):
    g = gen(5)
    shape_q = (2, 3, 7, 16) if heads_second else (2, 7, 3, 16)
    shape_k = (2, 3, 9, 16) if heads_second else (2, 9, 3, 16)
    q, k = (r64(g, *shape_q) * 2 + 0.5).requires_grad_(True), r64(g, *shape_k).requires_grad_(True)
    gq, gk = r64(g, *shape_q), r64(g, *shape_k)
    pe = oracle.rotary_table(10, 8).to(F64)
    qo, ko = oracle.ln_rope_fwd(q, k, pe, (4, 9), heads_second, 1e-5, F64)
    q2, k2 = oracle.rope_fwd(oracle.head_ln_fwd(q, 1e-5, F64), oracle.head_ln_fwd(k, 1e-5, F64), pe, (4, 9), heads_second, F64)
    torch.testing.assert_close(qo, q2, rtol=1e-13, atol=1e-14)
    torch.testing.assert_close(ko, k2, rtol=1e-13, atol=1e-14)
    dq_ad, dk_ad = torch.autograd.grad((qo, ko), (q, k), (gq, gk))
    dq, dk = oracle.ln_rope_bwd(gq, gk, q.detach(), k.detach(), pe, (4, 9), heads_second, 1e-5, F64)
    torch.testing.assert_close(dq, dq_ad, rtol=1e-9, atol=1e-12)
    torch.testing.assert_close(dk, dk_ad, rtol=1e-9, atol=1e-12)


# ------------------------------------------------------------------------------------------ attention
def brute_attention(q, k, v, bias, causal, scale):
    """python loops in fp64"""
    B, Tq, H, D = q.shape
    Tk = k.shape[1]
    o = torch.zeros(B, Tq, H, D, dtype=F64)
    lse = torch.zeros(B, H, Tq, dtype=F64)
    for b in range(B):
        for h in range(H):
            for i in range(Tq):
                s = []
                for j in range(Tk):
                    if causal and j > i:
                        s.append(-math.inf)
                        continue
                    x = sum(q[b, i, h, d].item() * k[b, j, h, d].item() for d in range(D)) * scale
                    if bias is not None:
                        bb = bias[b % bias.shape[0], h % bias.shape[1], i % bias.shape[2], j].item()
                        x += bb
                    s.append(x)
                m = max(s)
                z = sum(math.exp(x - m) for x in s)
                lse[b, h, i] = m + math.log(z)
                for j in range(Tk):
                    pj = math.exp(s[j] - m) / z
                    o[b, i, h] += pj * v[b, j, h]
    return o, lse


@pytest.mark.parametrize("bias_shape", [None, (1, 1, 5, 6), (2, 1, 5, 6), (1, 2, 5, 6), (2, 2, 5, 6), (2, 2, 1, 6)])
@pytest.mark.parametrize("causal", [False, True])
def test_attention_brute_force(bias_shape, causal):
    g = gen(6)
    q, k, v = r64(g, 2, 5, 2, 4), r64(g, 2, 6, 2, 4), r64(g, 2, 6, 2, 4)
    bias = None if bias_shape is None else r64(g, *bias_shape)
    o, lse = oracle.attention_fwd(q, k, v, bias, causal, None, F64)
    o_b, lse_b = brute_attention(q, k, v, bias, causal, 1 / math.sqrt(4))
    torch.testing.assert_close(o, o_b, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(lse.double(), lse_b, rtol=1e-6, atol=1e-6)
    # every broadcast form equals the materialised (B,h,Tq,Tk) form
    if bias is not None:
        o_full, _ = oracle.attention_fwd(q, k, v, bias.expand(2, 2, 5, 6).contiguous(), causal, None, F64)
        assert torch.equal(o, o_full)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_backward_against_autograd(causal):
    g = gen(7)
    q, k, v = (r64(g, 2, 7, 3, 8).requires_grad_(True), r64(g, 2, 9, 3, 8).requires_grad_(True),
               r64(g, 2, 9, 3, 8).requires_grad_(True))
    bias, do = r64(g, 2, 3, 7, 9), r64(g, 2, 7, 3, 8)
    bias[0, 0, :, 4] = -math.inf  # a masked key column
    s = torch.einsum("bthd,bshd->bhts", q, k) * 0.3 + bias
    if causal:
        s = s.masked_fill(torch.arange(7)[:, None] < torch.arange(9)[None, :], -math.inf)
    o = torch.einsum("bhts,bshd->bthd", torch.softmax(s, -1), v)
    ad = torch.autograd.grad(o, (q, k, v), do)
    got = oracle.attention_bwd(do, q.detach(), k.detach(), v.detach(), bias, causal, 0.3, F64)
    for a, r in zip(got, ad):
        torch.testing.assert_close(a, r, rtol=1e-9, atol=1e-12)
    assert torch.all(got[1][0, 4, 0] == 0) and torch.all(got[2][0, 4, 0] == 0)  # masked key: zero dk, dv rows
    o_f, lse = oracle.attention_fwd(q.detach(), k.detach(), v.detach(), bias, causal, 0.3, F64)
    torch.testing.assert_close(o_f, o.detach(), rtol=1e-11, atol=1e-13)
    torch.testing.assert_close(lse.double(), torch.logsumexp(s.detach(), -1), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("bias_shape", [(1, 1, 7, 9), (2, 1, 7, 9), (1, 3, 7, 9), (2, 3, 7, 9), (2, 3, 1, 9), (1, 1, 1, 9)])
@pytest.mark.parametrize("causal", [False, True])
def test_attention_bias_gradient_against_autograd(bias_shape, causal):
    g = gen(23)
    q, k, v, do = r64(g, 2, 7, 3, 8), r64(g, 2, 9, 3, 8), r64(g, 2, 9, 3, 8), r64(g, 2, 7, 3, 8)
    bias = r64(g, *bias_shape).requires_grad_(True)
    s = torch.einsum("bthd,bshd->bhts", q, k) * 0.3 + bias
    if causal:
        s = s.masked_fill(torch.arange(7)[:, None] < torch.arange(9)[None, :], -math.inf)
    o = torch.einsum("bhts,bshd->bthd", torch.softmax(s, -1), v)
    (db_ad,) = torch.autograd.grad(o, (bias,), do)
    got = oracle.attention_bwd(do, q, k, v, bias.detach(), causal, 0.3, F64, with_dbias=True)
    assert got[3].shape == bias.shape
    torch.testing.assert_close(got[3], db_ad, rtol=1e-9, atol=1e-12)


def test_attention_defaults_and_dead_rows():
    g = gen(8)
    q, k, v = r64(g, 1, 3, 1, 16), r64(g, 1, 4, 1, 16), r64(g, 1, 4, 1, 16)
    a, _ = oracle.attention_fwd(q, k, v, None, False, None, F64)
    b, _ = oracle.attention_fwd(q, k, v, None, False, 0.25, F64)   # 1/sqrt(16)
    c, _ = oracle.attention_fwd(q, k, v, None, False, 0.0, F64)    # 0.0 means "default" in the reference
    assert torch.equal(a, b) and torch.equal(a, c)
    bias = torch.zeros(1, 1, 3, 4, dtype=F64)
    bias[0, 0, 1] = -math.inf
    o, lse = oracle.attention_fwd(q, k, v, bias, False, None, F64)
    assert torch.all(o[0, 1] == 0) and lse[0, 0, 1] == -math.inf and not torch.isnan(o).any()
    dq, dk, dv = oracle.attention_bwd(r64(g, 1, 3, 1, 16), q, k, v, bias, False, None, F64)
    assert not any(torch.isnan(t).any() for t in (dq, dk, dv)) and torch.all(dq[0, 1] == 0)


# ------------------------------------------------------------------------------------------ attention_lowp
# attention_lowp is the error bar of the GPU attention tests (reference tests/test_flash_attn.py:44-62 with
# upcast=False, reorder_ops=True).  Two pins: in fp64 it is the same function as attention_fwd (a dropped bias, a
# wrong scale or mask fails), and in 16-bit types its error sits in a band around the rounding error of the
# result itself (an accidental upcast falls below the band, an extra source of error above it).
LOWP_BIASES = [None, (1, 1, 7, 9), (2, 1, 7, 9), (1, 3, 7, 9), (2, 3, 7, 9), (2, 3, 1, 9)]


@pytest.mark.parametrize("bias_shape", LOWP_BIASES)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("d", [8, 12])  # 1/sqrt(12) is not a power of two
def test_attention_lowp_is_attention_fwd_in_fp64(bias_shape, causal, d):
    g = gen(20)
    q, k, v = r64(g, 2, 7, 3, d), r64(g, 2, 9, 3, d), r64(g, 2, 9, 3, d)
    bias = None if bias_shape is None else r64(g, *bias_shape)
    o_ref, _ = oracle.attention_fwd(q, k, v, bias, causal, None, F64)
    o_lp = oracle.attention_lowp(q, k, v, bias, causal)
    assert o_lp.dtype == F64
    torch.testing.assert_close(o_lp, o_ref, rtol=1e-12, atol=1e-12)
    o_brute, _ = brute_attention(q, k, v, bias, causal, 1 / math.sqrt(d))
    torch.testing.assert_close(o_lp, o_brute, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_lowp_gradients_in_fp64(causal):
    """autograd through attention_lowp (what the GPU tests use as the gradient error bar) equals the closed-form
    backward"""
    g = gen(21)
    q, k, v = (r64(g, 2, 7, 3, 12).requires_grad_(True), r64(g, 2, 9, 3, 12).requires_grad_(True),
               r64(g, 2, 9, 3, 12).requires_grad_(True))
    bias, do = r64(g, 2, 3, 7, 9), r64(g, 2, 7, 3, 12)
    ad = torch.autograd.grad(oracle.attention_lowp(q, k, v, bias, causal), (q, k, v), do)
    got = oracle.attention_bwd(do, q.detach(), k.detach(), v.detach(), bias, causal, None, F64)
    for a, r in zip(got, ad):
        torch.testing.assert_close(a, r, rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 128, 128, 3, 64), (2, 97, 203, 3, 32), (1, 384, 384, 2, 128)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_attention_lowp_error_band(dtype, shape, with_bias):
    """N(0,1) inputs, no mask.  Measured over these cases: the output error of the low-precision run is 2.7-6.4
    times the error of rounding the exact result to the dtype (that ratio is 1 for a run that upcasts), and the
    gradient errors are 1.0-4.5 half-ulps of the largest gradient element (at most 0.5 for a run that upcasts)."""
    B, Tq, Tk, H, d = shape
    g = gen(22)
    q, k, v, do = (randn(g, B, T, H, d, dtype=dtype) for T in (Tq, Tk, Tk, Tq))
    bias = randn(g, B, H, Tq, Tk, dtype=dtype) if with_bias else None
    f = lambda t: None if t is None else t.float()
    exact, _ = oracle.attention_fwd(f(q), f(k), f(v), f(bias))                # fp32 in, fp32 out
    rounded, _ = oracle.attention_fwd(q, k, v, bias)                          # fp32 math, one rounding
    ql, kl, vl = (t.clone().requires_grad_(True) for t in (q, k, v))
    lowp = oracle.attention_lowp(ql, kl, vl, bias)
    assert lowp.dtype == dtype
    err = (lowp.float() - exact).abs().max().item()
    err_round = (rounded.float() - exact).abs().max().item()
    assert 2.0 * err_round <= err <= 10.0 * err_round, f"output error {err} vs rounding error {err_round}"
    half_ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    g_lp = torch.autograd.grad(lowp, (ql, kl, vl), do)
    g_ref = oracle.attention_bwd(do, q, k, v, bias)
    for a, r, n in zip(g_lp, g_ref, ("dq", "dk", "dv")):
        assert a.dtype == dtype
        rel = ((a.float() - r.float()).abs().max() / r.float().abs().max()).item() / half_ulp
        assert 0.7 <= rel <= 8.0, f"{n}: error of the low-precision gradient = {rel} half-ulps of its largest element"


# ------------------------------------------------------------------------------------------ tolerances
def test_tolerance_tables_match_reference_tests():
    """(rtol, atol) exactly as the reference's test files define them"""
    f32, f16, bf = torch.float32, torch.float16, torch.bfloat16
    assert oracle.get_tolerance(f32) == (1.3e-6, 1e-5) and oracle.get_tolerance(f16) == (1e-3, 1e-5)
    assert oracle.get_tolerance(bf) == (1.6e-2, 1e-5) and oracle.get_tolerance(bf, "rms") == (1.6e-2, 2e-5)
    assert oracle.get_tolerance(f16, "rope") == (1e-3, 1e-3) and oracle.get_tolerance(bf, "rope") == (1.6e-2, 1e-5)
    assert oracle.get_tolerance(f16, "ln_rope") == (1e-3, 1e-2) and oracle.get_tolerance(bf, "ln_rope") == (1.6e-2, 1e-3)
    with pytest.raises(ValueError):
        oracle.get_tolerance(torch.int32)
