"""The benchmark configurations at their full sizes.  The CPU oracle finishes these only on slices, so each
configuration is checked through (a) the oracle on a slice that the operator computes independently of the
rest (rows of a row operator, query rows of attention), and (b) properties that hold at any size: batch /
head permutation equivariance (bit-exact), key permutation invariance, V = const -> O = const, a constant
added to every logit moves only the LSE, the inner-product identities <dO, O> = <dV, V> and
<dQ, Q> = <dK, K>, linearity of the gradients in dO, exactly zero gradients for masked keys."""
import math

import pytest
import torch

from helpers import assert_close, gen, oracle, randn, to_gpu

pytestmark = pytest.mark.gpu


def _attn(q, k, v, bias, do, scale=None):
    from rgd_triton_amd import flash_attn_func

    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
    o, lse = flash_attn_func(qg, kg, vg, bias, False, scale, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
    return o.detach(), lse.detach(), dq, dk, dv


def _dot(a, b):
    return (a.double() * b.double()).sum().item()


def _rel(a, b):
    return abs(a - b) / max(abs(a), abs(b), 1e-30)


def _attention_properties(B, T, H, D, dtype, bias, seed, q_rows, exact_perm=True):
    """checks shared by configs 3, 4, 5; bias is a CPU tensor or None.  exact_perm=False: the launch splits the
    workgroups of its last grid round, so which (batch, head) items are summed in parts depends on their position and
    a permutation moves the last bits"""
    g = gen(seed)
    q, k, v, do = (randn(g, B, T, H, D, dtype=dtype) for _ in range(4))
    qg, kg, vg, dog = to_gpu(q, k, v, do)
    bg = None if bias is None else bias.to("cuda")
    o, lse, dq, dk, dv = _attn(qg, kg, vg, bg, dog)
    for t, n in ((o, "o"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert torch.isfinite(t.float()).all(), n

    # (a) oracle on a slice of query rows of one batch element (O, LSE and dQ of a query row depend on that row,
    # the keys and the values only)
    b0 = B - 1
    rows = torch.tensor(q_rows)
    bias_s = None
    if bias is not None:
        bb = b0 if bias.shape[0] == B else 0
        bias_s = bias[bb:bb + 1][:, :, rows]
    o_ref, lse_ref = oracle.attention_fwd(q[b0:b0 + 1, rows], k[b0:b0 + 1], v[b0:b0 + 1], bias_s)
    dq_ref = oracle.attention_bwd(do[b0:b0 + 1, rows], q[b0:b0 + 1, rows], k[b0:b0 + 1], v[b0:b0 + 1], bias_s)[0]
    ql, kl, vl = (t.clone().requires_grad_(True) for t in (q[b0:b0 + 1, rows], k[b0:b0 + 1], v[b0:b0 + 1]))
    o_pt = oracle.attention_lowp(ql, kl, vl, bias_s)
    dq_pt = torch.autograd.grad(o_pt, ql, do[b0:b0 + 1, rows])[0]
    err = (o[b0:b0 + 1, rows].cpu().float() - o_ref).abs().max().item()
    err_pt = (o_pt.detach().float() - o_ref).abs().max().item()
    assert err <= 2 * err_pt + 1e-5, f"o slice: {err} vs low-precision {err_pt}"
    torch.testing.assert_close(lse[b0:b0 + 1, :, rows].cpu(), lse_ref, rtol=1e-4, atol=1e-4)
    err = (dq[b0:b0 + 1, rows].cpu().float() - dq_ref.float()).abs().max().item()
    err_pt = (dq_pt.float() - dq_ref.float()).abs().max().item()
    assert err <= 2 * err_pt + 1e-5, f"dq slice: {err} vs low-precision {err_pt}"

    # (b1) inner-product identities of the exact gradients (fp32 accumulation on 16-bit tensors: 1 %)
    assert _rel(_dot(dog, o), _dot(dv, vg)) < 1e-2, (_dot(dog, o), _dot(dv, vg))
    assert _rel(_dot(dq, qg), _dot(dk, kg)) < 2e-2 or abs(_dot(dq, qg) - _dot(dk, kg)) < 1e-2 * math.sqrt(q.numel())

    # (b2) batch and head permutation: the same bits come out, permuted
    pb, ph = torch.randperm(B, generator=g), torch.randperm(H, generator=g)
    perm = lambda t: t[pb.to(t.device)][:, :, ph.to(t.device)]
    bg_p = None
    if bg is not None:
        bg_p = bg[pb.to("cuda")] if bg.shape[0] == B else bg
        bg_p = bg_p[:, ph.to("cuda")] if bg_p.shape[1] == H else bg_p
    o2, lse2, dq2, dk2, dv2 = _attn(perm(qg).contiguous(), perm(kg).contiguous(), perm(vg).contiguous(), bg_p,
                                    perm(dog).contiguous())
    for a, b_, n in ((o2, perm(o), "o"), (dq2, perm(dq), "dq"), (dk2, perm(dk), "dk"), (dv2, perm(dv), "dv")):
        if exact_perm:
            assert torch.equal(a, b_), f"batch/head permutation changed {n}"
        else:
            assert (a.float() - b_.float()).abs().max().item() <= 1e-2 * b_.float().abs().max().item(), n
    if exact_perm:
        assert torch.equal(lse2, lse[pb.to("cuda")][:, ph.to("cuda")])
    else:
        torch.testing.assert_close(lse2, lse[pb.to("cuda")][:, ph.to("cuda")], rtol=1e-5, atol=1e-5)

    # (b3) V = const -> O = const (rows of P sum to one); dV is linear in dO
    c = 0.375
    oc = _attn(qg, kg, torch.full_like(vg, c), bg, dog)[0]
    assert (oc.float() - c).abs().max().item() <= 4e-3, (oc.float() - c).abs().max().item()
    dv_a = _attn(qg, kg, vg, bg, dog * 0.5)[4]
    torch.testing.assert_close(dv_a.float() * 2, dv.float(), rtol=2e-2, atol=2e-2 * dv.float().abs().max().item())
    return qg, kg, vg, dog, bg, (o, lse, dq, dk, dv)


def test_config3_attention_full_size():
    B, T, H, D = 4, 4096, 16, 64
    qg, kg, vg, dog, _, (o, lse, dq, dk, dv) = _attention_properties(B, T, H, D, torch.bfloat16, None, 1003,
                                                                     list(range(0, 4096, 37)))
    # a constant added to every logit (vector bias) moves the LSE by that constant and nothing else
    cbias = torch.full((B, 1, 1, T), 1.5, dtype=torch.bfloat16, device="cuda")
    o2, lse2, dq2, dk2, dv2 = _attn(qg, kg, vg, cbias, dog)
    torch.testing.assert_close(lse2[..., :T], lse[..., :T] + 1.5, rtol=1e-4, atol=1e-4)
    assert (o2.float() - o.float()).abs().max().item() <= 2e-2
    # key permutation: O and dQ unchanged up to summation order, dK and dV permuted
    pk = torch.randperm(T, generator=gen(7)).to("cuda")
    o3, _, dq3, dk3, dv3 = _attn(qg, kg[:, pk].contiguous(), vg[:, pk].contiguous(), None, dog)
    assert (o3.float() - o.float()).abs().max().item() <= 2e-2
    scale = dq.float().abs().max().item()
    assert (dq3.float() - dq.float()).abs().max().item() <= 2e-2 * scale
    assert (dv3.float() - dv[:, pk].float()).abs().max().item() <= 2e-2 * dv.float().abs().max().item()
    assert (dk3.float() - dk[:, pk].float()).abs().max().item() <= 2e-2 * dk.float().abs().max().item()


def test_config4_attention_full_size_block_causal_bias():
    B, T, H, D = 2, 2048, 16, 128
    g = gen(1004)
    bias = 0.5 * torch.randn(B, H, T, T, generator=g)
    i = torch.arange(T)
    bias.masked_fill_((i[None, :] // 128) > (i[:, None] // 128), float("-inf"))
    bias = bias.to(torch.float16)
    qg, kg, vg, dog, bg, (o, lse, dq, dk, dv) = _attention_properties(B, T, H, D, torch.float16, bias, 2004,
                                                                     list(range(5, 2048, 61)))
    # the first 128 query rows see the first 128 keys only: the same numbers as attention over that corner
    oc, lsec, dqc, _, _ = _attn(qg[:, :128].contiguous(), kg[:, :128].contiguous(), vg[:, :128].contiguous(),
                                bg[:, :, :128, :128].contiguous(), dog[:, :128].contiguous())
    assert (oc.float() - o[:, :128].float()).abs().max().item() <= 2e-3
    torch.testing.assert_close(lsec[..., :128], lse[..., :128], rtol=1e-4, atol=1e-4)
    assert (dqc.float() - dq[:, :128].float()).abs().max().item() <= 2e-2 * dq.float().abs().max().item()
    # the last 128 keys are visible to the last 128 query rows only
    dk_tail = _attn(qg[:, -128:].contiguous(), kg, vg, bg[:, :, -128:].contiguous(), dog[:, -128:].contiguous())[3]
    assert (dk_tail[:, -128:].float() - dk[:, -128:].float()).abs().max().item() <= 2e-2 * dk.float().abs().max().item()


def test_config5_attention_full_size_padding_bias():
    B, T, H, D = 2, 4352, 24, 64
    g = gen(1005)
    bias = torch.zeros(B, 1, T, T)
    dead = []
    for b in range(B):
        d = T - 256 + torch.randperm(256, generator=g)[:26]
        bias[b, :, :, d] = float("-inf")
        dead.append(d)
    bias = bias.to(torch.bfloat16)
    qg, kg, vg, dog, bg, (o, lse, dq, dk, dv) = _attention_properties(B, T, H, D, torch.bfloat16, bias, 2005,
                                                                     list(range(3, 4352, 53)), exact_perm=False)
    for b in range(B):
        assert torch.all(dk[b, dead[b].to("cuda")] == 0) and torch.all(dv[b, dead[b].to("cuda")] == 0)
    # dropping the masked keys from K and V gives the same output
    keep = torch.ones(T, dtype=torch.bool)
    keep[dead[0]] = False
    keep = keep.to("cuda")
    o0 = _attn(qg[:1], kg[:1, keep].contiguous(), vg[:1, keep].contiguous(), None, dog[:1])[0]
    assert (o0.float() - o[:1].float()).abs().max().item() <= 2e-2


def test_config2_ln_rope_full_size():
    from rgd_triton_amd import FusedLNRoPE

    B, T, H, D = 8, 2048, 16, 64
    g = gen(2002)
    dt = torch.bfloat16
    q, k, gq, gk = (randn(g, B, T, H, D, dtype=dt) for _ in range(4))
    pe = oracle.rotary_table(T + 1, 32, 10000.0, dt)
    m = FusedLNRoPE()

    def run(q_, k_, gq_, gk_):
        qg, kg = to_gpu(q_, k_, requires_grad=True)
        qo, ko = m(qg, kg, pe.to("cuda"), seq_cutoff=(T, T), heads_second=False, eps=1e-5)
        dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq_.to("cuda"), gk_.to("cuda")))
        return qo.detach(), ko.detach(), dq, dk

    qo, ko, dq, dk = run(q, k, gq, gk)
    # oracle on a slice: the last batch element, every 16th token would need a strided table, so a token range
    b0, t0, t1 = B - 1, 1900, 2048
    pe_s = torch.cat([pe[:, t0:t1], pe[:, :1]], dim=1)  # rows t0..t1-1 (+1 spare row: T < P)
    sl = lambda t: t[b0:b0 + 1, t0:t1]
    qr, kr = oracle.ln_rope_fwd(sl(q), sl(k), pe_s, (t1 - t0, t1 - t0), False, 1e-5)
    dqr, dkr = oracle.ln_rope_bwd(sl(gq), sl(gk), sl(q), sl(k), pe_s, (t1 - t0, t1 - t0), False, 1e-5)
    for a, r, n in ((qo, qr, "qo"), (ko, kr, "ko"), (dq, dqr, "dq"), (dk, dkr, "dk")):
        assert_close(sl(a), r, dt, "ln_rope", n)
    # batch permutation: same bits, permuted
    pb = torch.randperm(B, generator=g)
    qo2, ko2, dq2, dk2 = run(q[pb], k[pb], gq[pb], gk[pb])
    pbg = pb.to("cuda")
    for a, b_, n in ((qo2, qo[pbg], "qo"), (ko2, ko[pbg], "ko"), (dq2, dq[pbg], "dq"), (dk2, dk[pbg], "dk")):
        assert torch.equal(a, b_), n
    # rotation keeps the norm of every (2i, 2i+1) pair, so a normalised row keeps |y|^2 = D * var / (var + eps)
    var = q.float().var(dim=-1, unbiased=False)
    want = (D * var / (var + 1e-5)).to("cuda")
    got = qo.float().pow(2).sum(-1)
    assert (got - want).abs().max().item() <= 0.03 * D
    # the LayerNorm gradient is orthogonal to constants and to the normalised row (before the rotation: use k with
    # the rotation switched off through the cutoff)
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo3, ko3 = m(qg, kg, pe.to("cuda"), seq_cutoff=(0, 0), heads_second=False, eps=1e-5)
    dq3, _ = torch.autograd.grad((qo3, ko3), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    assert dq3.float().sum(-1).abs().max().item() <= 0.05 * dq3.float().abs().max().item() * math.sqrt(D)


def test_config1_rmsnorm_full_size():
    from rgd_triton_amd import FusedRMSNorm

    g = gen(1001)
    x, dy = randn(g, 4, 1024, 1024), randn(g, 4, 1024, 1024)
    w = 1 + 0.1 * torch.randn(1024, generator=g)
    m = FusedRMSNorm(1024, eps=1e-6, device="cuda", dtype=torch.float32)
    with torch.no_grad():
        m.weight.copy_(w)
    xg = x.to("cuda").requires_grad_(True)
    y = m(xg)
    dx, dw = torch.autograd.grad(y, (xg, m.weight), dy.to("cuda"))
    assert_close(y, oracle.rms_fwd(x, w), torch.float32, name="y")
    dxr, dwr = oracle.rms_bwd(dy, x, w)
    assert_close(dx, dxr, torch.float32, name="dx")
    # dw sums 4096 rows: compare in relative terms of the column's magnitude
    torch.testing.assert_close(dw.cpu(), dwr, rtol=1e-4, atol=1e-3)


def test_config5_head_layernorm_full_size():
    from rgd_triton_amd import FusedHeadLayerNorm

    B, T, H, D = 2, 4352, 24, 64
    g = gen(3005)
    dt = torch.bfloat16
    q, k, gq, gk = (randn(g, B, T, H, D, dtype=dt) for _ in range(4))
    m = FusedHeadLayerNorm()
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo, ko = m(qg, kg, heads_second=False)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    sl = lambda t: t[1:2, 4000:4352]
    assert_close(sl(qo), oracle.head_ln_fwd(sl(q)), dt, name="qo")
    assert_close(sl(ko), oracle.head_ln_fwd(sl(k)), dt, name="ko")
    assert_close(sl(dq), oracle.head_ln_bwd(sl(gq), sl(q)), dt, name="dq")
    assert_close(sl(dk), oracle.head_ln_bwd(sl(gk), sl(k)), dt, name="dk")
    # every output row has zero mean and unit variance; every gradient row sums to zero
    assert qo.float().mean(-1).abs().max().item() <= 2e-2
    assert (qo.float().var(-1, unbiased=False) - 1).abs().max().item() <= 3e-2
    assert dq.float().sum(-1).abs().max().item() <= 0.05 * dq.float().abs().max().item() * math.sqrt(D)
    # shifting and scaling the input rows changes nothing (exactly representable factors)
    qo2, _ = m((qg.detach() * 2 + 4).to(dt), kg.detach(), heads_second=False)
    assert (qo2.float() - qo.float()).abs().max().item() <= 6e-2
