"""The operators inside the callers the reference describes: the README's Attention block
(README.md:36-60: qkv Linear -> unbind -> FusedHeadLayerNorm -> FlashAttention -> out_proj) and the
MMDiT-style joint block of benchmark configuration 5 (FusedRMSNorm2 on image+text streams -> projections ->
FusedHeadLayerNorm -> FlashAttention with a broadcast padding bias), forward and backward, against the
same block built from the CPU oracle's math with PyTorch autograd."""
import math

import pytest
import torch
import torch.nn as nn

from helpers import gen, oracle, randn

pytestmark = pytest.mark.gpu


class Attention(nn.Module):
    """README.md:36-60, verbatim structure"""

    def __init__(self, dim, n_heads, attn_op, head_norm):
        super().__init__()
        self.n_heads = n_heads
        self.head_dim = dim // n_heads
        self.qkv = nn.Linear(dim, dim * 3, bias=False)
        self.out_proj = nn.Linear(dim, dim)
        self.attn_op = attn_op
        self.head_norm = head_norm

    def forward(self, x, bias=None):
        B, T, C = x.shape
        q, k, v = self.qkv(x).view(B, T, 3, self.n_heads, self.head_dim).permute(2, 0, 1, 3, 4).unbind(dim=0)
        q, k = self.head_norm(q, k, heads_second=False)
        attn_out = self.attn_op(q, k, v, bias=bias)
        attn_out = attn_out.reshape(B, T, C)
        return self.out_proj(attn_out)


def ref_head_norm(q, k, heads_second=False, eps=1e-6):
    f = lambda t: torch.nn.functional.layer_norm(t.float(), (t.shape[-1],), None, None, eps).to(t.dtype)
    return f(q), f(k)


def ref_attention(q, k, v, bias=None, heads_per_chunk=4):
    """fp32 attention in plain PyTorch, a few heads at a time (the scores of all 24 heads of the full-size joint block
    would be 3.6 GB, several times over for autograd)"""
    d = q.shape[-1]
    outs = []
    for h0 in range(0, q.shape[2], heads_per_chunk):
        hs = slice(h0, h0 + heads_per_chunk)
        s = torch.einsum("bthd,bshd->bhts", q[:, :, hs].float(), k[:, :, hs].float()) / math.sqrt(d)
        if bias is not None:
            s = s + (bias if bias.shape[1] == 1 else bias[:, hs]).float()
        outs.append(torch.einsum("bhts,bshd->bthd", torch.softmax(s, -1), v[:, :, hs].float()))
    return torch.cat(outs, dim=2).to(q.dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("with_bias", [False, True])
def test_readme_attention_block(with_bias, dtype):
    from rgd_triton_amd import FlashAttention, FusedHeadLayerNorm

    torch.manual_seed(0)
    B, T, dim, heads = 2, 333, 512, 8
    blk = Attention(dim, heads, FlashAttention(), FusedHeadLayerNorm()).to("cuda", dtype)
    ref = Attention(dim, heads, ref_attention, ref_head_norm).to("cuda", dtype)
    ref.load_state_dict(blk.state_dict())
    g = gen(1)
    x = randn(g, B, T, dim, dtype=dtype).cuda()
    bias = (0.5 * torch.randn(B, 1, T, T, generator=g)).to(dtype).cuda() if with_bias else None
    dy = randn(g, B, T, dim, dtype=dtype).cuda()
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = blk(xa, bias), ref(xb, bias)
    ga = torch.autograd.grad(ya, [xa] + list(blk.parameters()), dy)
    gb = torch.autograd.grad(yb, [xb] + list(ref.parameters()), dy)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=5e-3, atol=5e-3)
    torch.testing.assert_close(ya, yb, **tol)
    for a, b in zip(ga, gb):
        scale = b.float().abs().max().item()
        torch.testing.assert_close(a.float() / scale, b.float() / scale, **tol)
    # the modules cached their launches, and toggling the cache does not change results
    assert blk.attn_op.cache.fwd is not None and blk.head_norm.cache.bwd is not None
    for m in blk.modules():
        if hasattr(m, "enable_cache"):
            m.enable_cache(False)
    assert torch.equal(blk(xa, bias), ya)


@pytest.mark.parametrize("size", ["reduced", "config5"])
def test_mmdit_joint_block_chain(size):
    """benchmark configuration 5 as a chain (the [image || text] joint sequence, -inf bias on ~10 % of the text keys per batch
    element, everything bf16), at a reduced size and at its real size (2 x (4096 + 256) tokens, 1536 channels, 24 heads
    of 64), forward and backward against the same chain in fp32 PyTorch on the CPU."""
    from rgd_triton_amd import FlashAttention, FusedHeadLayerNorm, FusedRMSNorm2

    g = gen(1005)
    dt = torch.bfloat16
    B, Ti, Tt, C, H, D = (2, 640, 96, 384, 6, 64) if size == "reduced" else (2, 4096, 256, 1536, 24, 64)
    img, txt = randn(g, B, Ti, C, dtype=dt), randn(g, B, Tt, C, dtype=dt)
    w1 = (1 + 0.1 * torch.randn(C, generator=g)).to(dt)
    w2 = (1 + 0.1 * torch.randn(C, generator=g)).to(dt)
    wqkv_i = (torch.randn(C, 3 * C, generator=g) / math.sqrt(C)).to(dt)
    wqkv_t = (torch.randn(C, 3 * C, generator=g) / math.sqrt(C)).to(dt)
    T = Ti + Tt
    bias = torch.zeros(B, 1, T, T)
    for b in range(B):
        dead = Ti + torch.randperm(Tt, generator=g)[: Tt // 10]
        bias[b, :, :, dead] = float("-inf")
    bias = bias.to(dt)
    do = randn(g, B, T, H, D, dtype=dt)

    def run(norm2, head_ln, attn, dev):
        i_, t_ = img.to(dev).requires_grad_(True), txt.to(dev).requires_grad_(True)
        a1, a2 = w1.to(dev).requires_grad_(True), w2.to(dev).requires_grad_(True)
        n1, n2 = norm2(i_, t_, a1, a2)
        qkv = torch.cat([n1 @ wqkv_i.to(dev), n2 @ wqkv_t.to(dev)], dim=1).view(B, T, 3, H, D)
        q, k, v = qkv.unbind(2)
        q, k = head_ln(q, k)
        o = attn(q, k, v, bias.to(dev))
        grads = torch.autograd.grad(o, (i_, t_, a1, a2), do.to(dev))
        return (o,) + grads

    norm = FusedRMSNorm2((C, C), elementwise_affine=False)
    fa, hl = FlashAttention(), FusedHeadLayerNorm()
    got = run(lambda a, b, c, d: norm(a, b, c, d), lambda q, k: hl(q, k, heads_second=False), lambda q, k, v, b: fa(q, k, v, bias=b), "cuda")

    def ref_norm2(a, b, c, d):
        f = lambda x, w: (torch.nn.functional.rms_norm(x.float(), (C,), None, 1e-6) * w.float()).to(dt)
        return f(a, c), f(b, d)

    ref = run(ref_norm2, lambda q, k: ref_head_norm(q, k), ref_attention, "cpu")
    for a, r, n in zip(got, ref, ("o", "d_img", "d_txt", "dw1", "dw2")):
        assert not torch.isnan(a).any(), n
        scale = r.float().abs().max().item()
        torch.testing.assert_close(a.cpu().float() / scale, r.float() / scale, rtol=3e-2, atol=3e-2, msg=lambda m: f"{n}: {m}")
