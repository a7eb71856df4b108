"""GPU parity of FlashAttention / flash_attn_func against the CPU oracle.  Counterpart of the
reference's tests/test_flash_attn.py: qkv :68-178, output :180-309, race :312-388,
bwd_overflow :391-451, bwd_transpose :454-513.  The acceptance rule is the reference's: the error
against the fp32 oracle may be at most a small multiple of the error of a low-precision PyTorch
evaluation of the same formula."""
import math

import pytest
import torch

from helpers import assert_repeats_bit_exact, gen, gpu_gen, oracle, randn, to_gpu

pytestmark = pytest.mark.gpu

HALF = [torch.float16, torch.bfloat16]


def make_bias(g, kind, B, H, Tq, Tk, dtype):
    shape = {"none": None, "static": (1, 1, Tq, Tk), "batch": (B, 1, Tq, Tk), "head": (1, H, Tq, Tk),
             "cube": (B, H, Tq, Tk), "vector": (B, H, 1, Tk)}[kind]
    return None if shape is None else randn(g, *shape, dtype=dtype)


def run_case(q, k, v, bias, do, causal=False, scale=None):
    """returns (o, lse, dq, dk, dv) from the GPU and the oracle's (o, lse, dq, dk, dv) + low-precision o"""
    from rgd_triton_amd import flash_attn_func

    qg, kg, vg = to_gpu(q, k, v, requires_grad=True)
    bg = None if bias is None else bias.to("cuda")
    o, lse = flash_attn_func(qg, kg, vg, bg, causal, scale, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to("cuda"))
    return (o, lse, dq, dk, dv)


def reference(q, k, v, bias, do, causal=False, scale=None):
    o_ref, lse_ref = oracle.attention_fwd(q, k, v, bias, causal, scale)
    g_ref = oracle.attention_bwd(do, q, k, v, bias, causal, scale)
    # the low-precision PyTorch run (upcast=False, reorder_ops=True) and its autograd gradients
    ql, kl, vl = (t.clone().requires_grad_(True) for t in (q, k, v))
    if scale is None:
        o_pt = oracle.attention_lowp(ql, kl, vl, bias, causal)
        g_pt = torch.autograd.grad(o_pt, (ql, kl, vl), do)
    else:
        o_pt, g_pt = None, None
    return o_ref, lse_ref, g_ref, o_pt, g_pt


def maxdiff(a, b):
    return (a.detach().cpu().float() - b.detach().float()).abs().max().item()


# Absolute backstop of every comparison, independent of the low-precision error bar: the error against the fp32
# oracle, in half-ulps of the tensor dtype at the scale of the largest reference element (of 1 for outputs
# smaller than that).  The kernels round P and dS once to the operand type and accumulate in fp32: 1-4 half-ulps.
ABS_HALF_ULPS = 12.0


def half_ulp(dtype):
    return 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11


def check(got, ref, Tq, out_mult=2, grad_mult=2, grad_add=0.0, name=""):
    o, lse, dq, dk, dv = got
    o_ref, lse_ref, g_ref, o_pt, g_pt = ref
    assert not torch.isnan(o).any() and not torch.isnan(dq).any() and not torch.isnan(dk).any() and not torch.isnan(dv).any()
    assert maxdiff(o, o_ref) <= out_mult * maxdiff(o_pt, o_ref) + 1e-5, f"{name} o: {maxdiff(o, o_ref)} vs {maxdiff(o_pt, o_ref)}"
    hu = ABS_HALF_ULPS * half_ulp(o.dtype)
    assert maxdiff(o, o_ref) <= hu * max(1.0, o_ref.float().abs().max().item()), f"{name} o: absolute error {maxdiff(o, o_ref)}"
    for a, r, pt, n in zip((dq, dk, dv), g_ref, g_pt, ("dq", "dk", "dv")):
        assert maxdiff(a, r) <= grad_mult * maxdiff(pt, r) + grad_add + 1e-5, f"{name} {n}: {maxdiff(a, r)} vs {maxdiff(pt, r)}"
        assert maxdiff(a, r) <= hu * max(1.0, r.float().abs().max().item()), f"{name} {n}: absolute error {maxdiff(a, r)}"
    fin = torch.isfinite(lse_ref)
    torch.testing.assert_close(lse[..., :Tq].cpu()[fin], lse_ref[fin], rtol=1e-4, atol=1e-4)
    assert torch.all(lse[..., Tq:] == 0)


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("bias_type", ["none", "static", "batch", "head", "cube"])
@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("seqlen", [14, 31, 97, 128, 200, 384, 768, 1025])
def test_flash_attn_qkv(seqlen, d, bias_type, dtype):
    """packed qkv (views with token stride 3*h*d), square attention, every bias broadcast form"""
    g = gen(0)
    B, H = (4, 9) if seqlen < 768 else (2, 5)
    qkv = randn(g, 3, B, seqlen, H, d, dtype=dtype)
    q, k, v = qkv.unbind(0)
    bias = make_bias(g, bias_type, B, H, seqlen, seqlen, dtype)
    do = randn(g, B, seqlen, H, d, dtype=dtype)
    check(run_case(q, k, v, bias, do), reference(q, k, v, bias, do), seqlen, name=f"qkv {bias_type}")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("bias_type", ["none", "static", "batch", "head", "cube"])
@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("Tq,Tk", [(113, 203), (128, 217), (113, 211), (108, 256), (256, 512), (512, 256),
                                    (1024, 1024), (1023, 1024), (1024, 1023), (239, 1), (1, 239), (2048, 2048)])
def test_flash_attn_output(Tq, Tk, d, bias_type, dtype):
    g = gen(0)
    # the CPU oracle dominates the run time: fewer (batch, head) pairs for the long sequences
    B, H = (2, 3) if Tq >= 1023 else (4, 9)
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype)
    do = randn(g, B, Tq, H, d, dtype=dtype)
    got = run_case(q, k, v, bias, do)
    if Tq < 2048:
        check(got, reference(q, k, v, bias, do), Tq, grad_mult=3, name=f"out {bias_type}")
        return
    # (2048, 2048): o, lse and dq of a query row depend on that row of q, do and the bias only, so the oracle checks
    # them on three bands of 128 query rows (first, one across the middle, the ragged end of the last block); dk and dv
    # sum over all query rows and are checked through the identities <dO,O> = <dV,V> and <dQ,Q> = <dK,K> and,
    # for one (batch, head), against the full oracle.
    o, lse, dq, dk, dv = got
    for r0 in (0, 960, 1920):
        rows = slice(r0, r0 + 128)
        bs = None if bias is None else bias[:, :, rows]
        ref = reference(q[:, rows], k, v, bs, do[:, rows])
        o_ref, lse_ref, g_ref, o_pt, g_pt = ref
        band = (o[:, rows], lse[..., rows], dq[:, rows], dk, dv)
        assert maxdiff(band[0], o_ref) <= 2 * maxdiff(o_pt, o_ref) + 1e-5, f"o rows {r0}"
        assert maxdiff(band[2], g_ref[0]) <= 3 * maxdiff(g_pt[0], g_ref[0]) + 1e-5, f"dq rows {r0}"
        hu = ABS_HALF_ULPS * half_ulp(dtype)
        assert maxdiff(band[0], o_ref) <= hu * max(1.0, o_ref.float().abs().max().item())
        assert maxdiff(band[2], g_ref[0]) <= hu * max(1.0, g_ref[0].float().abs().max().item())
        torch.testing.assert_close(band[1].cpu(), lse_ref, rtol=1e-4, atol=1e-4)
    f = lambda t: t.detach().double().cpu()
    tol = 2e-2 if dtype == torch.bfloat16 else 3e-3
    a, b_ = (f(do) * f(o)).sum(), (f(dv) * v.double()).sum()
    assert abs(a - b_) <= tol * max(abs(a), (f(do) * f(o)).abs().sum() * 0.01), "<dO,O> != <dV,V>"
    a, b_ = (f(dq) * q.double()).sum(), (f(dk) * k.double()).sum()
    assert abs(a - b_) <= tol * (f(dq) * q.double()).abs().sum() * 0.05, "<dQ,Q> != <dK,K>"
    one = lambda t: t[1:2, :, 2:3]
    bs = None if bias is None else bias[min(1, bias.shape[0] - 1):min(1, bias.shape[0] - 1) + 1,
                                        min(2, bias.shape[1] - 1):min(2, bias.shape[1] - 1) + 1]
    ref = reference(one(q), one(k), one(v), bs, one(do))
    check((one(o), lse[1:2, 2:3], one(dq), one(dk), one(dv)), ref, Tq, grad_mult=3, name=f"out {bias_type} (one head)")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("d", [40, 59, 80, 96, 111, 128, 8, 16])
@pytest.mark.parametrize("Tq,Tk", [(97, 131), (256, 128)])
def test_flash_attn_head_dims(Tq, Tk, d, dtype):
    """head dims that are not powers of two, including ones whose rows are not 16-byte aligned"""
    g = gen(1)
    q, k, v = randn(g, 2, Tq, 3, d, dtype=dtype), randn(g, 2, Tk, 3, d, dtype=dtype), randn(g, 2, Tk, 3, d, dtype=dtype)
    bias = make_bias(g, "cube", 2, 3, Tq, Tk, dtype)
    do = randn(g, 2, Tq, 3, d, dtype=dtype)
    check(run_case(q, k, v, bias, do), reference(q, k, v, bias, do), Tq, grad_mult=3, name=f"d={d}")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bias_type", ["none", "cube"])
@pytest.mark.parametrize("d", [40, 80, 112])
def test_flash_attn_padded_head_dim_long(d, bias_type, causal, dtype):
    """head dims made of whole 16-byte chunks but below the kernels' padded width, over enough tiles for the main
    loop; q/k/v/do are column slices of wider tensors whose other columns hold NaN, so a read past the end of a
    row (into the neighbouring columns) would show up in every output"""
    g = gen(7)
    B, H, Tq, Tk = 1, 2, 448, 520
    wide = lambda T: torch.full((B, T, H, d + 24), float("nan"), dtype=dtype)
    q, k, v, do = wide(Tq), wide(Tk), wide(Tk), wide(Tq)
    for t, T in ((q, Tq), (k, Tk), (v, Tk), (do, Tq)):
        t[..., 8:8 + d] = randn(g, B, T, H, d, dtype=dtype)
    qs, ks, vs, dos = (t[..., 8:8 + d] for t in (q, k, v, do))
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype)
    from rgd_triton_amd import flash_attn_func

    qg, kg, vg, dog = (t.cuda()[..., 8:8 + d] for t in (q, k, v, do))
    qg.requires_grad_(True), kg.requires_grad_(True), vg.requires_grad_(True)
    o, lse = flash_attn_func(qg, kg, vg, None if bias is None else bias.cuda(), causal, None, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), dog)
    qc, kc, vc, doc = (t.contiguous() for t in (qs, ks, vs, dos))
    check((o, lse, dq, dk, dv), reference(qc, kc, vc, bias, doc, causal), Tq, grad_mult=3, name=f"d={d}")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bias_type", ["none", "vector", "cube"])
@pytest.mark.parametrize("Tq,Tk", [(128, 128), (200, 200), (113, 203), (300, 150), (1, 64)])
def test_flash_attn_causal_vector_fp32bias(Tq, Tk, bias_type, causal, dtype):
    """API corners the reference implements but does not test: causal (top-left aligned), vector bias
    (.., 1, Tk), fp32 bias with 16-bit q"""
    g = gen(2)
    B, H, d = 2, 4, 64
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bias = make_bias(g, bias_type, B, H, Tq, Tk, torch.float32)
    do = randn(g, B, Tq, H, d, dtype=dtype)
    # the low-precision comparison run adds the bias in q's dtype
    ref = reference(q, k, v, bias, do, causal)
    if bias is not None:
        ref_lp = reference(q, k, v, bias.to(dtype), do, causal)
        ref = ref[:3] + ref_lp[3:]
    check(run_case(q, k, v, bias, do, causal), ref, Tq, grad_mult=3, grad_add=2e-3, name=f"causal={causal} {bias_type}")


@pytest.mark.parametrize("dtype", HALF)
def test_flash_attn_softmax_scale_and_lse(dtype):
    g = gen(3)
    q, k, v = randn(g, 2, 150, 4, 64, dtype=dtype), randn(g, 2, 90, 4, 64, dtype=dtype), randn(g, 2, 90, 4, 64, dtype=dtype)
    do = randn(g, 2, 150, 4, 64, dtype=dtype)
    got = run_case(q, k, v, None, do, scale=0.2)
    o_ref, lse_ref, g_ref, _, _ = reference(q, k, v, None, do, scale=0.2)
    tol = 2e-2 if dtype == torch.bfloat16 else 3e-3
    assert maxdiff(got[0], o_ref) <= tol
    torch.testing.assert_close(got[1][..., :150].cpu(), lse_ref, rtol=1e-4, atol=1e-4)
    for a, r in zip(got[2:], g_ref):
        assert maxdiff(a, r) <= 4 * tol
    assert got[1].shape == (2, 4, 192)


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("seqlen", [1, 2, 5, 17, 128])
def test_flash_attn_bwd_overflow(seqlen, dtype):
    """large-magnitude inputs (q x5, k and v x3), tests/test_flash_attn.py:391-451"""
    g = gen(4)
    B, H, d = 2, 5, 64
    q = randn(g, B, seqlen, H, d, dtype=dtype, scale=5.0)
    k, v = randn(g, B, seqlen, H, d, dtype=dtype, scale=3.0), randn(g, B, seqlen, H, d, dtype=dtype, scale=3.0)
    do = randn(g, B, seqlen, H, d, dtype=dtype)
    check(run_case(q, k, v, None, do), reference(q, k, v, None, do), seqlen, grad_mult=5, grad_add=1e-3, name="overflow")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("Tq,Tk", [(128, 128), (113, 203), (256, 512), (1, 239)])
def test_flash_attn_bwd_transpose(Tq, Tk, dtype):
    """non-contiguous upstream gradient and heads-first storage of q, k, v (tests/test_flash_attn.py:454-513)"""
    from rgd_triton_amd import flash_attn_func

    g = gen(5)
    B, H, d = 3, 4, 64
    q = randn(g, B, H, Tq, d, dtype=dtype).transpose(1, 2)
    k, v = randn(g, B, H, Tk, d, dtype=dtype).transpose(1, 2), randn(g, B, H, Tk, d, dtype=dtype).transpose(1, 2)
    do = randn(g, B, H, Tq, d, dtype=dtype).transpose(1, 2)
    qg = q.transpose(1, 2).contiguous().to("cuda").transpose(1, 2).requires_grad_(True)
    kg = k.transpose(1, 2).contiguous().to("cuda").transpose(1, 2).requires_grad_(True)
    vg = v.transpose(1, 2).contiguous().to("cuda").transpose(1, 2).requires_grad_(True)
    dog = do.transpose(1, 2).contiguous().to("cuda").transpose(1, 2)
    assert Tq == 1 or (not qg.is_contiguous() and not dog.is_contiguous())
    o, lse = flash_attn_func(qg, kg, vg, None, False, None, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), dog)
    check((o, lse, dq, dk, dv), reference(q, k, v, None, do), Tq, name="transpose")


def test_flash_attn_masked_bias_no_nan():
    """-inf in the bias: block-causal mask (blocks of 128, as benchmark configuration 4) and padded keys
    (as config 5).  dk/dv rows of fully masked keys are exactly zero; nothing is NaN."""
    g = gen(6)
    B, H, T, d = 2, 3, 384, 64
    dtype = torch.float16
    q, k, v = randn(g, B, T, H, d, dtype=dtype), randn(g, B, T, H, d, dtype=dtype), randn(g, B, T, H, d, dtype=dtype)
    do = randn(g, B, T, H, d, dtype=dtype)
    bias = (0.5 * torch.randn(B, H, T, T, generator=g)).to(dtype)
    i = torch.arange(T)
    bias.masked_fill_((i[None, :] // 128) > (i[:, None] // 128), float("-inf"))
    check(run_case(q, k, v, bias, do), reference(q, k, v, bias, do), T, grad_mult=3, name="block causal")
    pad = torch.zeros(B, 1, T, T)
    dead = torch.randperm(T, generator=g)[:40]
    pad[:, :, :, dead] = float("-inf")
    pad = pad.to(torch.bfloat16)
    qb, kb, vb, dob = (t.to(torch.bfloat16) for t in (q, k, v, do))
    got = run_case(qb, kb, vb, pad, dob)
    check(got, reference(qb, kb, vb, pad, dob), T, grad_mult=3, name="padded keys")
    assert torch.all(got[3][:, dead] == 0) and torch.all(got[4][:, dead] == 0)
    # a first key tile that is entirely -inf must not poison the running max
    first = torch.zeros(1, 1, T, T)
    first[..., :128] = float("-inf")
    got = run_case(qb, kb, vb, first.to(torch.bfloat16), dob)
    check(got, reference(qb, kb, vb, first.to(torch.bfloat16), dob), T, grad_mult=3, name="first tile masked")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("bias_dtype", ["same", "fp32"])
@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("block", [32, 64, 128, 96])
def test_flash_attn_masked_tiles(block, d, bias_dtype, dtype):
    """Blocks of -inf in the bias whose edges sit on, and off, the kernels' tile edges: the kernels leave out a block of
    logits when every bias value a wavefront holds for it is -inf, and the result must be what the full computation
    gives (block-diagonal + random visible blocks; ragged lengths so the last tiles are partial; one batch element has
    a (B,1,Q,K) broadcast row of NaN-free ordinary values so unmasked tiles sit next to masked ones)."""
    g = gen(9)
    B, H, Tq, Tk = 2, 3, 330, 420
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    do = randn(g, B, Tq, H, d, dtype=dtype)
    bt = torch.float32 if bias_dtype == "fp32" else dtype
    bias = (0.5 * torch.randn(B, H, Tq, Tk, generator=g))
    qi, ki = torch.arange(Tq) // block, torch.arange(Tk) // block
    visible = torch.rand(B, H, qi.max() + 1, ki.max() + 1, generator=g) < 0.4
    visible[..., 0] = True  # every query row keeps its first key block
    mask = ~visible[:, :, qi][:, :, :, ki]
    bias = bias.masked_fill(mask, float("-inf")).to(bt)
    ref = reference(q, k, v, bias, do)
    if bias_dtype == "fp32":  # the low-precision comparison run adds the bias in q's dtype
        ref = ref[:3] + reference(q, k, v, bias.to(dtype), do)[3:]
    got = run_case(q, k, v, bias, do)
    check(got, ref, Tq, grad_mult=3, grad_add=2e-3 if bias_dtype == "fp32" else 0.0, name=f"masked tiles {block}")
    # keys that no query of their (batch, head) sees get exactly zero gradients
    dead = mask.all(dim=2)  # (B, H, Tk)
    dk, dv = got[3].cpu().permute(0, 2, 1, 3), got[4].cpu().permute(0, 2, 1, 3)
    assert torch.all(dk[dead] == 0) and torch.all(dv[dead] == 0)


QUEUED_PATTERNS = ["block_causal_128", "block_causal_64", "block_anticausal", "diagonal_band", "random_blocks"]
QUEUED_CASES = ([(128, 1024, p, s) for p in QUEUED_PATTERNS for s in ("cube", "batch", "static", "cube_fp32")] +
                [(96, 1024, p, "batch") for p in QUEUED_PATTERNS] + [(128, 1000, p, "cube") for p in QUEUED_PATTERNS])


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("d,T,pattern,bias_shape", QUEUED_CASES)
def test_flash_attn_masked_tiles_queued_workgroups(d, T, pattern, bias_shape, dtype):
    """A launch with more workgroups than the chip holds at once first looks for the all -inf tiles at the end (forward,
    dQ) or the start (dK/dV) of each workgroup's loop and leaves them out of it; smaller launches do not.  Block-shaped
    masks in a launch of that size (24 x 4 heads x 8 row blocks), checked on one batch element against the oracle, and
    against the same batch element computed alone in a small launch (the tiles left out contribute exactly nothing:
    same bits, unless the small launch splits its workgroups along the keys)."""
    from rgd_triton_amd import flash_attn_func

    B, H, b0 = 24, 4, 13
    gg = torch.Generator(device="cuda").manual_seed(21)  # inputs this large are drawn on the GPU; the oracle gets one batch element
    qg, kg, vg, dog = (torch.randn(B, T, H, d, generator=gg, device="cuda").to(dtype) for _ in range(4))
    shape = {"cube": (B, H, T, T), "cube_fp32": (B, H, T, T), "batch": (B, 1, T, T), "static": (1, 1, T, T)}[bias_shape]
    bg = 0.5 * torch.randn(shape, generator=gg, device="cuda")
    i = torch.arange(T, device="cuda")
    if pattern == "block_causal_128":
        mask = (i[None, :] // 128) > (i[:, None] // 128)
    elif pattern == "block_causal_64":
        mask = (i[None, :] // 64) > (i[:, None] // 64)
    elif pattern == "block_anticausal":  # the first keys are the hidden ones
        mask = (i[None, :] // 128) < (i[:, None] // 128)
    elif pattern == "diagonal_band":  # hidden tiles at both ends of every loop
        mask = ((i[None, :] // 128) - (i[:, None] // 128)).abs() > 1
    else:
        vis = torch.rand(shape[0], shape[1], (T + 127) // 128, (T + 127) // 128, generator=gg, device="cuda") < 0.35
        vis[..., 3] = True
        mask = ~vis[:, :, i // 128][:, :, :, i // 128]
    bg = bg.masked_fill(mask, float("-inf")).to(torch.float32 if bias_shape == "cube_fp32" else dtype)
    one = slice(b0, b0 + 1)
    q, k, v, do = (t[one].cpu() for t in (qg, kg, vg, dog))
    bias_one = (bg if bg.shape[0] == 1 else bg[one]).cpu()

    def run(sl):
        qs, ks, vs = (t[sl].detach().requires_grad_(True) for t in (qg, kg, vg))
        bs = bg if bg.shape[0] == 1 else bg[sl]
        o, lse = flash_attn_func(qs, ks, vs, bs, False, None, return_lse=True)
        return (o.detach(), lse.detach()) + torch.autograd.grad(o, (qs, ks, vs), dog[sl])

    big = run(slice(0, B))
    ref = reference(q, k, v, bias_one, do)
    if bias_shape == "cube_fp32":  # the low-precision comparison run adds the bias in q's dtype
        ref = ref[:3] + reference(q, k, v, bias_one.to(dtype), do)[3:]
    check(tuple(t[one] for t in big), ref, T, grad_mult=3, grad_add=2e-3 if bias_shape == "cube_fp32" else 0.0,
          name=f"{pattern} in a queued launch")
    small = run(one)
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10  # one rounding step of the output type
    for a, b_, n in zip(big, small, ("o", "lse", "dq", "dk", "dv")):
        a, b_ = a[one].float().nan_to_num(posinf=0.0, neginf=0.0), b_.float().nan_to_num(posinf=0.0, neginf=0.0)
        assert (a - b_).abs().max().item() <= (1e-5 if n == "lse" else 1.01 * ulp) * max(1.0, b_.abs().max().item()), n


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("bias_shape", ["cube", "batch", "vector"])
@pytest.mark.parametrize("pattern", ["block_causal", "block_anticausal", "band", "random_blocks", "none_hidden", "all_hidden_rows"])
@pytest.mark.parametrize("d,Tq,Tk", [(128, 700, 520), (96, 384, 640), (128, 128, 1024), (128, 1100, 96)])
def test_flash_attn_bwd_key_ranges(d, Tq, Tk, pattern, bias_shape, dtype):
    """With room in the workspace, the dQ launch of rgd_attn_bwd notes which keys each 32 query rows can see (bias above
    -inf) and the dK/dV launch leaves the query tiles before the first and after the last such rows out of each key
    block's loop.  Through the C ABI: a workspace with room for delta and the notes only (no split), the full workspace
    (split items note all keys) and a workspace without room for the notes must give the same dK and dV bit for bit
    (the steps left out add exact zeros), and the oracle's values."""
    import ctypes
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    g = gen(31)
    B, H = 2, 3
    q, do = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tq, H, d, dtype=dtype)
    k, v = randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    shape = {"cube": (B, H, Tq, Tk), "batch": (B, 1, Tq, Tk), "vector": (B, H, 1, Tk)}[bias_shape]
    bias = 0.5 * torch.randn(shape, generator=g)
    qi, ki = torch.arange(shape[2])[:, None] // 64, torch.arange(Tk)[None, :] // 64
    qs = qi * ((Tk + 63) // 64) // ((Tq + 63) // 64)  # the row block's place on the key axis: every row sees some key
    if pattern == "block_causal":
        mask = ki > qs
    elif pattern == "block_anticausal":
        mask = ki < qs - 1
    elif pattern == "band":
        mask = (ki - qs).abs() > 1
    elif pattern == "random_blocks":
        vis = torch.rand(shape[0], shape[1], (shape[2] + 63) // 64, (Tk + 63) // 64, generator=g) < 0.3
        vis[..., 1] = True
        mask = ~vis[:, :, torch.arange(shape[2]) // 64][:, :, :, torch.arange(Tk) // 64]
    elif pattern == "none_hidden":
        mask = torch.zeros(shape[2], Tk, dtype=torch.bool)
    else:  # whole row blocks see nothing, the others everything
        mask = ((qi % 3) == 1).expand(shape[2], Tk)
    if bias_shape == "vector":  # a vector can only hide keys from every query
        mask = (ki % 3 == 1) if pattern not in ("none_hidden",) else torch.zeros(1, Tk, dtype=torch.bool)
    bias = bias.masked_fill(mask, float("-inf")).to(dtype)
    qg, kg, vg, dog, bg = (t.cuda() for t in (q, k, v, do, bias))
    code = _hip.dtype_code(dtype)
    be = bg.expand(B, H, Tq, Tk)
    kind = _hip.BIAS_VECTOR if bias_shape == "vector" else _hip.BIAS_MATRIX
    bdesc = _hip.Tensor4(be.data_ptr(), be.stride(0), be.stride(1), be.stride(2))
    st = _hip.stream_ptr(qg.device)
    scale = 1.0 / math.sqrt(d)
    tqr = lib.rgd_attn_seqlen_q_rounded(Tq)
    delta_bytes = B * H * tqr * 4
    notes_bytes = B * H * ((Tq + 127) // 128) * 4 * 2 * 4
    full_b = lib.rgd_attn_bwd_workspace(B, H, Tq, Tk, d, 1)
    assert full_b >= delta_bytes + notes_bytes + 16
    o = torch.empty_like(qg)
    lse = torch.empty(B, H, tqr, dtype=torch.float32, device="cuda")
    t = {n: _hip.t4(x, False) for n, x in dict(q=qg, k=kg, v=vg, do=dog, o=o).items()}
    assert lib.rgd_attn_fwd(B, H, Tq, Tk, d, t["q"], t["k"], t["v"], bdesc, kind, code, t["o"], lse.data_ptr(), code, 0, scale,
                            None, None, 0, st) == 0, lib.rgd_last_error()

    def run(bws_bytes):
        dq, dk, dv = torch.empty_like(qg), torch.empty_like(kg), torch.empty_like(vg)
        bws = torch.empty(bws_bytes, dtype=torch.uint8, device="cuda")
        tt = {n: _hip.t4(x, False) for n, x in dict(dq=dq, dk=dk, dv=dv).items()}
        rc = lib.rgd_attn_bwd(B, H, Tq, Tk, d, t["do"], t["q"], t["k"], t["v"], t["o"], lse.data_ptr(), bdesc, kind, code,
                              tt["dq"], tt["dk"], tt["dv"], None, code, 0, scale, 1, None, bws.data_ptr(), bws_bytes, st)
        assert rc == 0, lib.rgd_last_error()
        torch.cuda.synchronize()
        return dq, dk, dv

    plain = run(delta_bytes)                       # no notes, no split
    noted = run(delta_bytes + notes_bytes + 16)    # notes, no room to split
    full = run(full_b)                             # notes, and whatever the library splits
    for a, b_, n in zip(noted, plain, ("dq", "dk", "dv")):
        assert torch.equal(a, b_), f"{n} differs when the dK/dV launch uses the noted key ranges"
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for a, b_, n in zip(full, plain, ("dq", "dk", "dv")):
        assert maxdiff(a, b_.cpu()) <= 1.01 * ulp * max(b_.float().abs().max().item(), 1.0), n
    g_ref = oracle.attention_bwd(do, q, k, v, bias, False, None)
    for a, n in zip(noted, ("dq", "dk", "dv")):
        assert not torch.isnan(a).any(), n
    if pattern == "all_hidden_rows" and bias_shape != "vector":
        # the low-precision PyTorch run gives NaN for a row that sees nothing: absolute bound instead
        hidden = ((torch.arange(Tq) // 64) % 3) == 1
        assert torch.all(noted[0][:, hidden.cuda()] == 0)
        for a, r, n in zip(noted, g_ref, ("dq", "dk", "dv")):
            assert maxdiff(a, r) <= ABS_HALF_ULPS * half_ulp(dtype) * max(1.0, r.float().abs().max().item()), n
        return
    ql, kl, vl = (x.clone().requires_grad_(True) for x in (q, k, v))
    g_pt = torch.autograd.grad(oracle.attention_lowp(ql, kl, vl, bias, False), (ql, kl, vl), do)
    for a, r, pt, n in zip(noted, g_ref, g_pt, ("dq", "dk", "dv")):
        assert maxdiff(a, r) <= 3 * maxdiff(pt, r) + 1e-5, f"{n}: {maxdiff(a, r)} vs {maxdiff(pt, r)}"


def test_flash_attn_fully_masked_row_gives_zero():
    g = gen(7)
    q, k, v = (randn(g, 1, 70, 2, 32, dtype=torch.float16) for _ in range(3))
    bias = torch.zeros(1, 1, 70, 70, dtype=torch.float16)
    bias[0, 0, 5, :] = float("-inf")
    do = randn(g, 1, 70, 2, 32, dtype=torch.float16)
    o, lse, dq, dk, dv = run_case(q, k, v, bias, do)
    assert torch.all(o[0, 5] == 0) and torch.all(torch.isinf(lse[0, :, 5])) and torch.all(dq[0, 5] == 0)
    for t in (o, dq, dk, dv):
        assert not torch.isnan(t).any()


RACE_PAIRS = [(1, 239), (239, 1), (3, 799), (799, 3), (1024, 128), (97, 97), (128, 128), (200, 200), (256, 256),
              (257, 257), (384, 384), (512, 512), (768, 768), (1024, 1024)]


@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("bias_type", ["none", "cube"])
@pytest.mark.parametrize("Tq,Tk", RACE_PAIRS + [(113, 203), (1023, 1024)])
def test_flash_attn_race_condition(Tq, Tk, bias_type, d):
    """The reference's determinism test at its own strength (tests/test_flash_attn.py:312-388): batch 60, 4 heads,
    its 14 (Tq, Tk) pairs (plus two ragged ones), 250 repeats of forward + backward.  The reference allows dq to
    move by rounding noise (:368,383); here o, lse, dq, dk and dv must all reproduce bit for bit."""
    from rgd_triton_amd import flash_attn_func

    g = gpu_gen(8)
    dtype = torch.float16
    B, H = 60, 4
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype)
    do = randn(g, B, Tq, H, d, dtype=dtype).to("cuda")
    qg, kg, vg = to_gpu(q, k, v, requires_grad=True)
    bg = None if bias is None else bias.to("cuda")

    def step():
        o, lse = flash_attn_func(qg, kg, vg, bg, False, None, return_lse=True)
        return (o, lse, *torch.autograd.grad(o, (qg, kg, vg), do))

    assert_repeats_bit_exact(step, ("o", "lse", "dq", "dk", "dv"))


DETERMINISTIC_PAIRS = [(1, 239), (3, 799), (127, 512), (127, 513), (113, 203), (128, 217), (113, 211), (108, 256),
                       (256, 512), (1023, 1024)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bias_type", ["none", "cube"])
@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("swap_sq_sk", [False, True])
@pytest.mark.parametrize("Tq,Tk", DETERMINISTIC_PAIRS)
def test_flash_attn_deterministic(Tq, Tk, swap_sq_sk, d, bias_type, dtype):
    """The test the reference carries but skips ("Determinism not implemented", tests/test_flash_attn.py:546-609):
    batch 4, 9 heads, its ten (Tq, Tk) pairs both ways round, 50 repeats of the backward of one forward; dq, dk and
    dv must have the bits of the first run every time.  The two-kernel backward writes every gradient element once."""
    from rgd_triton_amd import flash_attn_func

    if swap_sq_sk:
        Tq, Tk = Tk, Tq
    g = gen(14)
    B, H = 4, 9
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype)
    do = randn(g, B, Tq, H, d, dtype=dtype).to("cuda")
    qg, kg, vg = to_gpu(q, k, v, requires_grad=True)
    bg = None if bias is None else bias.to("cuda")
    out = flash_attn_func(qg, kg, vg, bg, False, None, return_lse=False)
    assert_repeats_bit_exact(lambda: torch.autograd.grad(out, (qg, kg, vg), do, retain_graph=True), ("dq", "dk", "dv"), iters=50)


@pytest.fixture
def one_pass():
    """the one-pass backward (dQ through fp32 atomics) for the duration of a test"""
    from rgd_triton_amd import set_attention_backward

    prev = set_attention_backward("one_pass")
    yield
    set_attention_backward(prev)


ONE_PASS_PAIRS = [(113, 203), (128, 217), (256, 512), (512, 256), (1023, 1024), (1, 239), (239, 1), (64, 64)]
# every pair and bias form at the two main head dims; the padded and odd head dims on three pairs and two bias forms
ONE_PASS_CASES = ([(tq, tk, d, b) for tq, tk in ONE_PASS_PAIRS for d in (32, 64) for b in ("none", "batch", "cube", "vector")] +
                  [(tq, tk, d, b) for tq, tk in ((113, 203), (1023, 1024), (1, 239)) for d in (40, 59, 16) for b in ("none", "cube")])


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Tq,Tk,d,bias_type", ONE_PASS_CASES)
def test_flash_attn_one_pass_backward(Tq, Tk, d, bias_type, causal, dtype, one_pass):
    """The one-pass form of the backward (head dims up to 64): same acceptance rule as the two-kernel form."""
    g = gen(12)
    B, H = (2, 3) if Tq >= 1023 else (3, 5)
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype)
    do = randn(g, B, Tq, H, d, dtype=dtype)
    check(run_case(q, k, v, bias, do, causal), reference(q, k, v, bias, do, causal), Tq, grad_mult=3, name="one pass")


def test_flash_attn_one_pass_matches_two_kernel(one_pass):
    """strided qkv views, a -inf mask and a fully masked query row through both forms: dK and dV agree to the rounding
    of the different summation order, dQ too; wider heads fall back to the two-kernel form"""
    from rgd_triton_amd import flash_attn_func, set_attention_backward

    g = gen(13)
    B, T, H, d = 2, 300, 4, 64
    qkv = randn(g, 3, B, T, H, d, dtype=torch.bfloat16)
    bias = 0.5 * torch.randn(B, 1, T, T, generator=g)
    bias[:, :, :, 130:200] = float("-inf")
    bias[0, 0, 7, :] = float("-inf")
    bias = bias.to(torch.bfloat16)
    do = randn(g, B, T, H, d, dtype=torch.bfloat16)
    got = run_case(*qkv.unbind(0), bias, do)
    set_attention_backward("two_kernel")
    ref = run_case(*qkv.unbind(0), bias, do)
    set_attention_backward("one_pass")
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    for a, r, n in zip(got[2:], ref[2:], ("dq", "dk", "dv")):
        assert not torch.isnan(a).any()
        assert maxdiff(a, r.cpu()) <= 2.0 ** -7 * max(1.0, r.float().abs().max().item()), n
    assert torch.all(got[2][0, 7] == 0) and torch.all(got[3][:, 130:200] == 0) and torch.all(got[4][:, 130:200] == 0)
    big = [randn(g, 1, 70, 2, 128, dtype=torch.float16) for _ in range(4)]
    check(run_case(big[0], big[1], big[2], None, big[3]), reference(big[0], big[1], big[2], None, big[3]), 70, name="d=128")


@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("bias_type", ["none", "cube"])
@pytest.mark.parametrize("Tq,Tk", RACE_PAIRS)
def test_flash_attn_race_condition_one_pass(Tq, Tk, bias_type, d, one_pass):
    """The reference's determinism test under its own rule (tests/test_flash_attn.py:312-388), for the one-pass form:
    o, lse, dk and dv reproduce bit for bit over 250 repeats; dq, which is accumulated with atomics, may move by
    the rounding noise the reference allows, atol = 2 * max|(dq + 0.3 - 0.3) - dq|."""
    from rgd_triton_amd import flash_attn_func

    g = gpu_gen(8)
    dtype = torch.float16
    B, H = 60, 4
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype)
    do = randn(g, B, Tq, H, d, dtype=dtype).to("cuda")
    qg, kg, vg = to_gpu(q, k, v, requires_grad=True)
    bg = None if bias is None else bias.to("cuda")
    dq_runs = []

    def step():
        o, lse = flash_attn_func(qg, kg, vg, bg, False, None, return_lse=True)
        dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
        if len(dq_runs) < 2 or len(dq_runs) % 25 == 0:
            dq_runs.append(dq.clone())
        else:
            dq_runs.append(None)
        return (o, lse, dk, dv)

    assert_repeats_bit_exact(step, ("o", "lse", "dk", "dv"))
    dq0 = dq_runs[0]
    atol = 2 * ((dq0 + 0.3 - 0.3) - dq0).abs().max().item()
    for dq in dq_runs[1:]:
        if dq is not None:
            assert torch.allclose(dq, dq0, atol=atol, rtol=0), f"dq moved by {(dq - dq0).abs().max().item()} (allowed {atol})"


def test_flash_attn_module_errors_and_cache():
    from rgd_triton_amd import FlashAttention, flash_attn_func

    m = FlashAttention()
    assert m.cache.fwd is None and m.cache.bwd is None and m.cache.bwd_odot is None
    q = torch.randn(1, 64, 2, 64, device="cuda", dtype=torch.float16, requires_grad=True)
    o = m(q, q, q)
    o.sum().backward()
    assert m.cache.fwd is not None and m.cache.bwd is not None and m.cache.bwd_odot is not None
    # a different shape and bias kind through the same cache must not reuse anything stale
    q2 = torch.randn(2, 100, 2, 32, device="cuda", dtype=torch.float16)
    b2 = torch.randn(2, 2, 100, 100, device="cuda", dtype=torch.float16)
    o2 = m(q2, q2, q2, bias=b2)
    o2_ref, _ = oracle.attention_fwd(q2.cpu(), q2.cpu(), q2.cpu(), b2.cpu())
    assert maxdiff(o2, o2_ref) < 5e-3
    with pytest.raises(AssertionError, match="Only support fp16 and bf16"):
        flash_attn_func(q.float(), q.float(), q.float())
    big = torch.randn(1, 8, 1, 256, device="cuda", dtype=torch.float16)
    with pytest.raises(AssertionError, match="head dimensions up to 128"):
        flash_attn_func(big, big, big)
    with pytest.raises(RuntimeError, match="Last 2 dimensions of bias"):
        flash_attn_func(q, q, q, torch.zeros(1, 1, 3, 64, device="cuda", dtype=torch.float16))


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("bias_dtype", ["same", "fp32"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bias_type", ["static", "batch", "head", "cube", "vector"])
@pytest.mark.parametrize("d,Tq,Tk", [(64, 113, 203), (32, 200, 130), (128, 256, 320), (59, 97, 64), (64, 1, 239)])
def test_flash_attn_bias_gradient(d, Tq, Tk, bias_type, causal, bias_dtype, dtype):
    """The gradient of the bias (the reference refuses it, flash_attn_triton_cached.py:1107): dS = P * (dP - delta) of
    every pair, summed over the dimensions the bias broadcasts, against the oracle's closed form (pinned by fp64
    autograd).  The other gradients are unchanged by asking for it."""
    from rgd_triton_amd import flash_attn_func

    g = gen(14)
    B, H = 2, 3
    q, k, v = randn(g, B, Tq, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype), randn(g, B, Tk, H, d, dtype=dtype)
    bt = torch.float32 if bias_dtype == "fp32" else dtype
    bias = make_bias(g, bias_type, B, H, Tq, Tk, torch.float32)
    bias[..., Tk // 3] = float("-inf")  # a masked key: zero gradient there
    bias = bias.to(bt)
    do = randn(g, B, Tq, H, d, dtype=dtype)
    qg, kg, vg = to_gpu(q, k, v, requires_grad=True)
    bg = bias.cuda().requires_grad_(True)
    o = flash_attn_func(qg, kg, vg, bg, causal)
    dq, dk, dv, db = torch.autograd.grad(o, (qg, kg, vg, bg), do.cuda())
    dq2, dk2, dv2 = torch.autograd.grad(flash_attn_func(qg, kg, vg, bg.detach(), causal), (qg, kg, vg), do.cuda())
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)
    ref = oracle.attention_bwd(do, q, k, v, bias, causal, None, with_dbias=True)[3]
    assert db.shape == bias.shape and db.dtype == bias.dtype and not torch.isnan(db).any()
    assert torch.all(db[..., Tk // 3] == 0)
    # Error model: an element is a sum of `terms` values dS = P * (dP - delta), each rounded to the operand type (a few
    # half-ulps of the largest |dS|), and delta = rowsum(O * dO) is formed from the O the forward stored, i.e. rounded
    # to the tensor type as in the reference's kernel (flash_attn_triton_cached.py:249-292), while the oracle keeps O
    # in fp32: that moves dP - delta by about half an ulp of |O| |dO| ~ sqrt(d).
    terms = max(1, (B * H * Tq * Tk) // ref.numel())
    scale = oracle.attention_bwd(do, q, k, v, bias.expand(B, H, Tq, Tk).contiguous(), causal, None,
                                 with_dbias=True)[3].float().abs().max().item()
    allowed = half_ulp(dtype) * (4 * scale + d ** 0.5) * terms ** 0.5
    assert maxdiff(db, ref) <= allowed, f"dbias error {maxdiff(db, ref)} (allowed {allowed}, scale {scale}, {terms} terms)"


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bias_type", ["static", "batch", "head", "vector"])
def test_flash_attn_bias_gradient_in_chunks(bias_type, causal, monkeypatch):
    """A bias that broadcasts over heads (else: over the batch) has its gradient formed in chunks of heads (batch
    elements) that fit a bounded buffer.  With the bound forced down to one head / one batch element per chunk, dq, dk
    and dv are the unchunked ones bit for bit, and the bias gradient differs only in how its fp32 sum is grouped."""
    from rgd_triton_amd import flash_attn_func, functional

    g = gen(15)
    B, H, Tq, Tk, d, dtype = 3, 5, 150, 200, 64, torch.bfloat16
    q, k, v, do = (randn(g, B, T, H, d, dtype=dtype).cuda() for T in (Tq, Tk, Tk, Tq))
    bias = make_bias(g, bias_type, B, H, Tq, Tk, dtype).cuda().requires_grad_(True)
    qg, kg, vg = (t.requires_grad_(True) for t in (q, k, v))

    def grads():
        return torch.autograd.grad(flash_attn_func(qg, kg, vg, bias, causal), (qg, kg, vg, bias), do)

    whole = grads()
    monkeypatch.setattr(functional, "_DBIAS_CHUNK_BYTES", 1)
    chunked = grads()
    for a, b in zip(whole[:3], chunked[:3]):
        assert torch.equal(a, b)
    assert chunked[3].shape == bias.shape and chunked[3].dtype == bias.dtype
    scale = whole[3].float().abs().max().item()
    assert maxdiff(chunked[3], whole[3].cpu()) <= 2 * half_ulp(dtype) * scale


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("B,H,T,d,with_bias,mode", [(1, 2, 2048, 64, False, 1), (1, 3, 1536, 128, True, 1), (2, 5, 1100, 32, True, 1),
                                                    (1, 2, 2048, 64, False, 2), (2, 5, 1100, 32, True, 2)])
def test_flash_attn_split_workgroups(B, H, T, d, with_bias, mode, dtype):
    """With a workspace the library splits the workgroups of a partly filled last round (here: a grid far
    smaller than the chip) along their inner loop and merges fp32 partial results.  Through the C ABI: the
    split run must agree with the unsplit run (no workspace / a workspace that only holds delta) to fp32
    regrouping accuracy, must be bit-reproducible, and both must pass the oracle check."""
    import ctypes
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    g = gen(11)
    q, k, v, do = (randn(g, B, T, H, d, dtype=dtype) for _ in range(4))
    bias = make_bias(g, "batch", B, H, T, T, dtype) if with_bias else None
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    code = _hip.dtype_code(dtype)
    if bias is None:
        bdesc, bk, bd = _hip.Tensor4(None, 0, 0, 0), _hip.BIAS_NONE, _hip.RGD_F32
    else:
        bg = bias.cuda()
        be = bg.expand(B, H, T, T)
        bdesc, bk, bd = _hip.Tensor4(be.data_ptr(), be.stride(0), be.stride(1), be.stride(2)), _hip.BIAS_MATRIX, code
    st = _hip.stream_ptr(qg.device)
    scale = 1.0 / math.sqrt(d)
    tqr = lib.rgd_attn_seqlen_q_rounded(T)
    delta_bytes = B * H * tqr * 4
    full_f, full_b = lib.rgd_attn_fwd_workspace(B, H, T, T, d), lib.rgd_attn_bwd_workspace(B, H, T, T, d, mode)
    assert full_b > delta_bytes

    def run(fws_bytes, bws_bytes):
        o, dq, dk, dv = (torch.empty_like(qg) for _ in range(4))
        lse = torch.empty(B, H, tqr, dtype=torch.float32, device="cuda")
        fws = torch.empty(max(fws_bytes, 16), dtype=torch.uint8, device="cuda")
        bws = torch.empty(bws_bytes, dtype=torch.uint8, device="cuda")
        t = {n: _hip.t4(x, False) for n, x in dict(q=qg, k=kg, v=vg, do=dog, o=o, dq=dq, dk=dk, dv=dv).items()}
        rc = lib.rgd_attn_fwd(B, H, T, T, d, t["q"], t["k"], t["v"], bdesc, bk, bd, t["o"], lse.data_ptr(), code, 0, scale,
                              None, fws.data_ptr() if fws_bytes else None, fws_bytes, st)
        assert rc == 0, lib.rgd_last_error()
        rc = lib.rgd_attn_bwd(B, H, T, T, d, t["do"], t["q"], t["k"], t["v"], t["o"], lse.data_ptr(), bdesc, bk, bd, t["dq"],
                              t["dk"], t["dv"], None, code, 0, scale, mode, None, bws.data_ptr(), bws_bytes, st)
        assert rc == 0, lib.rgd_last_error()
        torch.cuda.synchronize()
        return o, lse, dq, dk, dv

    # unsplit: a workspace that holds only what the form requires (delta; dq_accum too for the one-pass form)
    need = delta_bytes if mode == 1 else delta_bytes * (1 + (32 if d <= 32 else 64))
    plain = run(0, need)
    split = run(full_f, full_b)
    again = run(full_f, full_b)
    for a, b_, n in zip(split, again, ("o", "lse", "dq", "dk", "dv")):
        if n == "dq" and mode == 2:  # accumulated with atomics: rounding noise only
            assert maxdiff(a, b_.cpu()) <= 2.0 ** -7 * max(1.0, b_.float().abs().max().item())
            continue
        assert torch.equal(a, b_), f"{n}: the split run is not reproducible"
    # same math, other summation grouping: agreement far inside one rounding step of the output type
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for a, b_, n in zip(split, plain, ("o", "lse", "dq", "dk", "dv")):
        scale_n = b_.float().abs().max().item()
        assert maxdiff(a, b_.cpu()) <= (1e-5 if n == "lse" else 1.01 * ulp) * max(scale_n, 1.0), n
    # on a grid this much smaller than the chip the split really happens: regrouped fp32 sums differ in the
    # last bit of some of the thousands of LSE rows (the third case is left to the library's cost model)
    if B * H <= 3:
        assert not torch.equal(split[1], plain[1])
    ref = reference(q, k, v, bias, do)
    check(split, ref, T, grad_mult=3, name="split")
    check(plain, ref, T, grad_mult=3, name="unsplit")
