"""GPU parity of FusedRMSNorm2 / triton_fused_rms_func_fn.  Counterpart of the reference's
tests/test_fused_rms.py (parity :139-211, seqdiff with different widths :213-328, race :331-)."""
import pytest
import torch

from helpers import DTYPES, assert_close, assert_repeats_bit_exact, gen, gpu_gen, oracle, randn, to_gpu

pytestmark = pytest.mark.gpu


def _run(B, T1, T2, C1, C2, dtype, unique_bw, seed=0, eps=1e-6):
    from rgd_triton_amd import triton_fused_rms_func_fn

    g = gen(seed)
    x1, x2 = randn(g, B, T1, C1, dtype=dtype), randn(g, B, T2, C2, dtype=dtype)
    w1 = (1 + 0.1 * torch.randn((B, 1, C1) if unique_bw else (C1,), generator=g)).to(dtype)
    w2 = (1 + 0.1 * torch.randn((B, 1, C2) if unique_bw else (C2,), generator=g)).to(dtype)
    d1, d2 = randn(g, B, T1, C1, dtype=dtype), randn(g, B, T2, C2, dtype=dtype)
    x1g, x2g, w1g, w2g = to_gpu(x1, x2, w1, w2, requires_grad=True)
    y1, y2 = triton_fused_rms_func_fn(x1g, x2g, w1g, w2g, eps)
    grads = torch.autograd.grad((y1, y2), (x1g, x2g, w1g, w2g), (d1.to("cuda"), d2.to("cuda")))
    ref = (oracle.rms_fwd(x1, w1, eps), oracle.rms_fwd(x2, w2, eps)) + oracle.rms_bwd(d1, x1, w1, eps) + \
        oracle.rms_bwd(d2, x2, w2, eps)
    got = (y1, y2, grads[0], grads[2], grads[1], grads[3])
    return got, ref


def _check(got, ref, dtype, rows1, rows2, C1, C2):
    names = ("y1", "y2", "dx1", "dw1", "dx2", "dw2")
    scales = (1, 1, 1, 3 * rows1 * C1 ** 0.5, 1, 3 * rows2 * C2 ** 0.5)
    for a, r, n, s in zip(got, ref, names, scales):
        assert a.shape == r.shape and a.dtype == r.dtype, n
        assert_close(a, r, dtype, "rms", n, atol_scale=s)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("unique_bw", [False, True])
@pytest.mark.parametrize("C", [32, 97, 384, 1023, 1536])
@pytest.mark.parametrize("T", [31, 384])
def test_fused_rms_norm(T, C, unique_bw, dtype):
    B = 4
    got, ref = _run(B, T, T, C, C, dtype, unique_bw)
    rows = T if unique_bw else B * T
    _check(got, ref, dtype, rows, rows, C, C)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("unique_bw", [False, True])
@pytest.mark.parametrize("C,dfactor", [(32, -0.75), (97, -0.3), (384, 0.2), (510, 0.6), (1023, 1.0), (24, -0.75)])
@pytest.mark.parametrize("T1,T2", [(31, 11), (23, 138), (113, 203), (1023, 1024), (1, 239), (239, 1)])
def test_fused_rms_norm_seqdiff(T1, T2, C, dfactor, unique_bw, dtype):
    """different sequence lengths and different widths (C2 = C*(1+dfactor)) for the two tensors"""
    B = 3
    C2 = max(1, int(C * (1 + dfactor)))
    got, ref = _run(B, T1, T2, C, C2, dtype, unique_bw, seed=3)
    _check(got, ref, dtype, T1 if unique_bw else B * T1, T2 if unique_bw else B * T2, C, C2)


def test_fused_equals_single():
    """virtual tensor: op2(x1, x2) == (op1(x1), op1(x2)) bit for bit, forward and dx"""
    from rgd_triton_amd import triton_fused_rms_func_fn, triton_rms_func_fn

    g = gen(11)
    x1, x2 = randn(g, 2, 300, 1536, dtype=torch.bfloat16), randn(g, 2, 77, 1536, dtype=torch.bfloat16)
    w1 = (1 + 0.1 * torch.randn(1536, generator=g)).to(torch.bfloat16)
    w2 = (1 + 0.1 * torch.randn(1536, generator=g)).to(torch.bfloat16)
    d1, d2 = randn(g, 2, 300, 1536, dtype=torch.bfloat16), randn(g, 2, 77, 1536, dtype=torch.bfloat16)
    x1g, x2g, w1g, w2g = to_gpu(x1, x2, w1, w2, requires_grad=True)
    y1, y2 = triton_fused_rms_func_fn(x1g, x2g, w1g, w2g)
    f = torch.autograd.grad((y1, y2), (x1g, x2g), (d1.to("cuda"), d2.to("cuda")))
    s1 = triton_rms_func_fn(x1g, w1g)
    s2 = triton_rms_func_fn(x2g, w2g)
    (g1,) = torch.autograd.grad(s1, x1g, d1.to("cuda"))
    (g2,) = torch.autograd.grad(s2, x2g, d2.to("cuda"))
    assert torch.equal(y1, s1) and torch.equal(y2, s2)
    assert torch.equal(f[0], g1) and torch.equal(f[1], g2)


def test_fused_rms_config5_and_module():
    """Benchmark configuration 5a: image (2,4096,1536) + text (2,256,1536) bf16 through the Module."""
    from rgd_triton_amd import FusedRMSNorm2

    g = gen(1005)
    img, txt = randn(g, 2, 4096, 1536, dtype=torch.bfloat16), randn(g, 2, 256, 1536, dtype=torch.bfloat16)
    w1 = (1 + 0.1 * torch.randn(1536, generator=g)).to(torch.bfloat16)
    w2 = (1 + 0.1 * torch.randn(1536, generator=g)).to(torch.bfloat16)
    d1, d2 = randn(g, 2, 4096, 1536, dtype=torch.bfloat16), randn(g, 2, 256, 1536, dtype=torch.bfloat16)
    m = FusedRMSNorm2((1536, 1536), eps=1e-6, device="cuda", dtype=torch.bfloat16)
    assert sorted(m.state_dict().keys()) == ["weight1", "weight2"]
    with torch.no_grad():
        m.weight1.copy_(w1)
        m.weight2.copy_(w2)
    ig, tg = to_gpu(img, txt, requires_grad=True)
    y1, y2 = m(ig, tg)
    grads = torch.autograd.grad((y1, y2), (ig, tg, m.weight1, m.weight2), (d1.to("cuda"), d2.to("cuda")))
    ref = (oracle.rms_fwd(img, w1), oracle.rms_fwd(txt, w2)) + oracle.rms_bwd(d1, img, w1) + oracle.rms_bwd(d2, txt, w2)
    _check((y1, y2, grads[0], grads[2], grads[1], grads[3]), ref, torch.bfloat16, 8192, 512, 1536, 1536)
    with pytest.raises(AssertionError, match="requires 2 int dims"):
        FusedRMSNorm2(1536)


RACE_PAIRS = [(1, 239), (239, 1), (3, 799), (799, 3), (1024, 128), (97, 97), (128, 128), (200, 200), (256, 256),
              (257, 257), (384, 384), (512, 512), (768, 768), (1024, 1024)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("unique_bw", [True, False])
@pytest.mark.parametrize("C,dfactor", [(63, -0.75), (122, 0.2), (384, 0.6), (384, -0.3), (740, -0.3), (1023, 1.0)])
@pytest.mark.parametrize("T1,T2", RACE_PAIRS)
def test_fused_rms_norm_race_condition(T1, T2, C, dfactor, unique_bw, dtype):
    """The reference's race test (tests/test_fused_rms.py:331-): batch 60, its 14 length pairs, 250 repeats, on five
    of its nine widths (one of them with two ratios) and all five of its width ratios; every output and gradient must reproduce bit for bit."""
    from rgd_triton_amd import triton_fused_rms_func_fn

    g = gpu_gen(13)
    B, C2 = 60, max(1, int(C * (1 + dfactor)))
    x1, x2 = randn(g, B, T1, C, dtype=dtype), randn(g, B, T2, C2, dtype=dtype)
    w1 = randn(g, *((B, 1, C) if unique_bw else (C,)), dtype=dtype, scale=0.1, shift=1.0)
    w2 = randn(g, *((B, 1, C2) if unique_bw else (C2,)), dtype=dtype, scale=0.1, shift=1.0)
    d1, d2 = randn(g, B, T1, C, dtype=dtype), randn(g, B, T2, C2, dtype=dtype)
    a = to_gpu(x1, x2, w1, w2, requires_grad=True)

    def step():
        y = triton_fused_rms_func_fn(*a)
        return (*y, *torch.autograd.grad(y, a, (d1, d2)))

    assert_repeats_bit_exact(step, ("y1", "y2", "dx1", "dx2", "dw1", "dw2"))
