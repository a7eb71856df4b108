"""Empty inputs: zero tokens, zero batch, one empty stream of a two-stream operator, attention without keys or
without queries.  Every operator returns tensors of the right shape without a launch error, forward and backward;
what a non-empty part of the call computes is checked against the oracle."""
import pytest
import torch

from helpers import assert_close, gen, oracle, randn

pytestmark = pytest.mark.gpu

DT = torch.bfloat16


def _leaf(*shape, dtype=DT):
    return torch.randn(*shape, device="cuda").to(dtype).requires_grad_(True)


@pytest.mark.parametrize("B,T", [(2, 0), (0, 5), (0, 0)])
def test_rmsnorm_and_l2_empty(B, T):
    from rgd_triton_amd import triton_norm_func_fn, triton_rms_func_fn

    C = 96
    x, w = _leaf(B, T, C), _leaf(C)
    y = triton_rms_func_fn(x, w, 1e-6)
    assert y.shape == x.shape
    dx, dw = torch.autograd.grad(y, (x, w), torch.empty_like(y))
    assert dx.shape == x.shape and dw.shape == w.shape
    assert torch.all(dw == 0)
    z = triton_norm_func_fn(x, 1e-6)
    assert z.shape == x.shape
    (dx,) = torch.autograd.grad(z, (x,), torch.empty_like(z))
    assert dx.shape == x.shape
    torch.cuda.synchronize()


def test_fused_rmsnorm2_one_empty_stream():
    """an MMDiT block without text tokens: the image stream is still normalised"""
    from rgd_triton_amd import triton_fused_rms_func_fn

    g = gen(3)
    x1, x2 = randn(g, 2, 37, 192, dtype=DT), torch.empty(2, 0, 64, dtype=DT)
    w1, w2 = 1 + 0.1 * randn(g, 192, dtype=DT), 1 + 0.1 * randn(g, 64, dtype=DT)
    dy1 = randn(g, 2, 37, 192, dtype=DT)
    a = [t.cuda().requires_grad_(True) for t in (x1, x2, w1, w2)]
    y1, y2 = triton_fused_rms_func_fn(a[0], a[1], a[2], a[3], 1e-6)
    assert y2.shape == x2.shape
    assert_close(y1, oracle.rms_fwd(x1, w1), DT, "rms", "y1")
    dx1, dx2, dw1, dw2 = torch.autograd.grad((y1, y2), a, (dy1.cuda(), torch.empty_like(y2)))
    ref_dx, ref_dw = oracle.rms_bwd(dy1, x1, w1)
    assert_close(dx1, ref_dx, DT, "rms", "dx1")
    assert_close(dw1, ref_dw, DT, "rms", "dw1", atol_scale=3 * 74 * 192 ** 0.5)
    assert dx2.shape == x2.shape and torch.all(dw2 == 0)


@pytest.mark.parametrize("Tq,Tk", [(0, 7), (9, 0), (0, 0)])
def test_head_ops_empty_stream(Tq, Tk):
    from rgd_triton_amd import triton_fused_ln_func_fn, triton_fused_ln_rope_fn, triton_rope_fn

    B, H, D, R = 2, 3, 64, 32
    g = gen(5)
    qc, kc = randn(g, B, Tq, H, D, dtype=DT), randn(g, B, Tk, H, D, dtype=DT)
    pos = oracle.rotary_table(16, R).to(DT)
    for fn, ref in ((lambda q, k: triton_fused_ln_func_fn(q, k, False), lambda x: oracle.head_ln_fwd(x)),
                    (lambda q, k: triton_rope_fn(q, k, pos.cuda(), None, False), None),
                    (lambda q, k: triton_fused_ln_rope_fn(q, k, pos.cuda(), None, False), None)):
        q, k = qc.cuda().requires_grad_(True), kc.cuda().requires_grad_(True)
        qo, ko = fn(q, k)
        assert qo.shape == q.shape and ko.shape == k.shape
        dq, dk = torch.autograd.grad((qo, ko), (q, k), (torch.ones_like(qo), torch.ones_like(ko)))
        assert dq.shape == q.shape and dk.shape == k.shape
        if ref is not None:
            if Tq:
                assert_close(qo, ref(qc), DT, name="qo")
            if Tk:
                assert_close(ko, ref(kc), DT, name="ko")
    torch.cuda.synchronize()


def test_attention_without_keys_or_queries():
    from rgd_triton_amd import flash_attn_func

    B, H, D = 2, 3, 64
    # no keys: every row's softmax is over nothing, the output is 0 and the gradients are 0 / empty
    q, k, v = _leaf(B, 5, H, D), _leaf(B, 0, H, D), _leaf(B, 0, H, D)
    o, lse = flash_attn_func(q, k, v, None, False, None, return_lse=True)
    assert o.shape == q.shape and torch.all(o == 0)
    assert torch.all(lse[..., :5] == -float("inf"))
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), torch.ones_like(o))
    assert torch.all(dq == 0) and dk.shape == k.shape and dv.shape == v.shape
    # no queries: dK and dV are zero
    q, k, v = _leaf(B, 0, H, D), _leaf(B, 6, H, D), _leaf(B, 6, H, D)
    o = flash_attn_func(q, k, v)
    assert o.shape == q.shape
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), torch.empty_like(o))
    assert dq.shape == q.shape and torch.all(dk == 0) and torch.all(dv == 0)
    # no batch
    q, k, v = _leaf(0, 4, H, D), _leaf(0, 6, H, D), _leaf(0, 6, H, D)
    o = flash_attn_func(q, k, v)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), torch.empty_like(o))
    assert o.shape == q.shape and dk.shape == k.shape
    torch.cuda.synchronize()
