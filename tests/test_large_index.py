"""Tensors with more than 2^31 elements: element offsets have to be 64-bit everywhere.  Inputs are generated on
the GPU from closed formulas (a CPU generator would take minutes), and the slices that lie beyond the 2^31-element
mark are checked against the CPU oracle."""
import pytest
import torch

from helpers import assert_close, oracle

pytestmark = pytest.mark.gpu


def _pattern(shape, device, dtype, a, b, mod, scale, chunk=1 << 27):
    """x[i] = ((i * a + b) mod `mod`) / mod * scale - scale / 2 over the flat index i (int64 arithmetic)"""
    n = 1
    for d in shape:
        n *= d
    out = torch.empty(n, dtype=dtype, device=device)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        i = torch.arange(s, e, device=device, dtype=torch.int64)
        out[s:e] = (((i * a + b) % mod).to(torch.float32) / mod * scale - scale / 2).to(dtype)
    return out.view(*shape)


def test_rmsnorm_beyond_2g_elements():
    from rgd_triton_amd import triton_rms_func_fn

    B, T, C = 2, 280000, 4096  # 2.29e9 elements per tensor
    dt = torch.bfloat16
    x = _pattern((B, T, C), "cuda", dt, 7919, 13, 1009, 4.0)
    dy = _pattern((B, T, C), "cuda", dt, 104729, 5, 2003, 2.0)
    w = (1 + 0.1 * torch.sin(torch.arange(C, dtype=torch.float32))).to(dt).cuda()
    xg = x.requires_grad_(True)
    wg = w.clone().requires_grad_(True)
    y = triton_rms_func_fn(xg, wg, 1e-6)
    dx, dw = torch.autograd.grad(y, (xg, wg), dy)
    for b0, t0 in ((0, 0), (1, T - 64), (1, 140000)):  # flat offsets 0, ~2.29e9, ~1.72e9
        xs, dys = x[b0:b0 + 1, t0:t0 + 64].detach().cpu(), dy[b0:b0 + 1, t0:t0 + 64].cpu()
        assert_close(y[b0:b0 + 1, t0:t0 + 64], oracle.rms_fwd(xs, w.cpu()), dt, name=f"y {b0},{t0}")
        assert_close(dx[b0:b0 + 1, t0:t0 + 64], oracle.rms_bwd(dys, xs, w.cpu())[0], dt, name=f"dx {b0},{t0}")
    # dw over all 560000 rows: fp32 sums of the same products on the GPU, in chunks
    acc = torch.zeros(C, dtype=torch.float64, device="cuda")
    for b0 in range(B):
        for t0 in range(0, T, 20000):
            xf = x[b0, t0:t0 + 20000].detach().float()
            xh = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)
            acc += (xh * dy[b0, t0:t0 + 20000].float()).sum(0).double()
    ref = acc.float()
    assert (dw.float() - ref).abs().max().item() <= 8e-3 * ref.abs().max().item() + 1.0


def test_head_layernorm_beyond_2g_elements():
    from rgd_triton_amd import triton_fused_ln_func_fn

    B, T, H, D = 2, 70000, 256, 64  # 2.29e9 elements per tensor
    dt = torch.bfloat16
    q = _pattern((B, T, H, D), "cuda", dt, 6007, 3, 811, 4.0)
    k = _pattern((B, T, H, D), "cuda", dt, 7919, 11, 1013, 4.0)
    qo, ko = triton_fused_ln_func_fn(q, k, False)
    for b0, t0 in ((0, 0), (1, T - 8), (1, 40000)):
        qs, ks = q[b0:b0 + 1, t0:t0 + 8].cpu(), k[b0:b0 + 1, t0:t0 + 8].cpu()
        assert_close(qo[b0:b0 + 1, t0:t0 + 8], oracle.head_ln_fwd(qs), dt, name=f"qo {b0},{t0}")
        assert_close(ko[b0:b0 + 1, t0:t0 + 8], oracle.head_ln_fwd(ks), dt, name=f"ko {b0},{t0}")


def test_attention_bias_beyond_2g_elements():
    from rgd_triton_amd import flash_attn_func

    B, T, H, D = 1, 47104, 1, 32  # bias (1,1,T,T): 2.22e9 elements
    dt = torch.bfloat16
    q = _pattern((B, T, H, D), "cuda", dt, 7919, 13, 1009, 2.0)
    k = _pattern((B, T, H, D), "cuda", dt, 6007, 3, 811, 2.0)
    v = _pattern((B, T, H, D), "cuda", dt, 104729, 5, 2003, 2.0)
    do = _pattern((B, T, H, D), "cuda", dt, 3571, 7, 503, 2.0)
    bias = _pattern((1, 1, T, T), "cuda", dt, 48271, 17, 4099, 6.0)
    qg, kg, vg = (t.requires_grad_(True) for t in (q, k, v))
    o, lse = flash_attn_func(qg, kg, vg, bias, False, None, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
    # query rows on both sides of the 2^31-element mark of the bias (row 45591) and at the end
    rows = torch.tensor([0, 1, 63, 64, 45590, 45591, 45592, 46000, T - 2, T - 1])
    qs, bs, dos = q[:, rows].detach().cpu(), bias[:, :, rows].cpu(), do[:, rows].cpu()
    kc, vc = k.detach().cpu(), v.detach().cpu()
    o_ref, lse_ref = oracle.attention_fwd(qs, kc, vc, bs)
    dq_ref = oracle.attention_bwd(dos, qs, kc, vc, bs)[0]
    ql = qs.clone().requires_grad_(True)
    o_pt = oracle.attention_lowp(ql, kc, vc, bs)
    dq_pt = torch.autograd.grad(o_pt, ql, dos)[0]
    err, err_pt = (o[:, rows].cpu().float() - o_ref).abs().max().item(), (o_pt.detach().float() - o_ref).abs().max().item()
    assert err <= 2 * err_pt + 1e-5, f"o: {err} vs {err_pt}"
    torch.testing.assert_close(lse[:, :, rows].cpu(), lse_ref, rtol=1e-4, atol=1e-4)
    err, err_pt = (dq[:, rows].cpu().float() - dq_ref.float()).abs().max().item(), (dq_pt.float() - dq_ref.float()).abs().max().item()
    assert err <= 2 * err_pt + 1e-5, f"dq: {err} vs {err_pt}"
    # dK / dV see every bias row: the inner-product identities tie them to O and dQ
    dot = lambda a, b: (a.double() * b.double()).sum().item()
    assert abs(dot(do, o) - dot(dv, v)) <= 1e-2 * max(abs(dot(do, o)), 1.0)
    assert abs(dot(dq, q) - dot(dk, k)) <= 2e-2 * max(abs(dot(dq, q)), abs(dot(dk, k)), 1.0)
