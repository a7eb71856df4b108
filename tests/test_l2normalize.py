"""GPU parity of L2Normalize / FusedL2Normalize2.  Counterpart of the reference's
tests/test_l2normalize.py and tests/test_fused_l2normalize.py (inputs scaled x100, :41-45)."""
import pytest
import torch

from helpers import DTYPES, assert_close, assert_close_allow_inf, assert_repeats_bit_exact, gen, gpu_gen, oracle, randn, to_gpu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [32, 63, 97, 122, 257, 384, 510, 740, 1023, 2048, 4097, 6144, 16384])
@pytest.mark.parametrize("T", [14, 200, 1024])
def test_l2_norm(T, C, dtype):
    from rgd_triton_amd import triton_norm_func_fn

    g = gen(0)
    x = randn(g, 4, T, C, dtype=dtype, scale=100.0)
    dy = randn(g, 4, T, C, dtype=dtype)
    xg = to_gpu(x, requires_grad=True)
    y = triton_norm_func_fn(xg, 1e-6)
    (dx,) = torch.autograd.grad(y, xg, dy.to("cuda"))
    assert_close(y, oracle.l2_fwd(x, 1e-6), dtype, name="y")
    assert_close_allow_inf(dx, oracle.l2_bwd(dy, x, 1e-6), dtype, name="dx")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [16392, 20001, 40000])
def test_l2_norm_streamed_rows(C, dtype):
    """rows beyond the register-resident limit: two-pass streaming kernel, any width"""
    from rgd_triton_amd import triton_norm_func_fn

    g = gen(C)
    x = randn(g, 2, 23, C, dtype=dtype, scale=100.0)
    dy = randn(g, 2, 23, C, dtype=dtype)
    xg = to_gpu(x, requires_grad=True)
    y = triton_norm_func_fn(xg, 1e-6)
    (dx,) = torch.autograd.grad(y, xg, dy.to("cuda"))
    assert_close(y, oracle.l2_fwd(x, 1e-6), dtype, name="y")
    assert_close_allow_inf(dx, oracle.l2_bwd(dy, x, 1e-6), dtype, name="dx")


@pytest.mark.parametrize("dtype", DTYPES)
def test_l2_clamped_rows(dtype):
    """rows shorter than eps (including all-zero rows) take the 1/eps branch, forward and backward"""
    from rgd_triton_amd import L2Normalize

    g = gen(1)
    x = randn(g, 2, 16, 128, dtype=dtype)
    x[0, :4] = 0
    x[1, 4:8] *= 1e-4
    dy = randn(g, 2, 16, 128, dtype=dtype)
    xg = to_gpu(x, requires_grad=True)
    eps = 1e-2
    y = L2Normalize()(xg, eps=eps)
    (dx,) = torch.autograd.grad(y, xg, dy.to("cuda"))
    assert torch.all(y[0, :4] == 0)
    assert_close(y, oracle.l2_fwd(x, eps), dtype, name="y")
    assert_close_allow_inf(dx, oracle.l2_bwd(dy, x, eps), dtype, name="dx")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,dfactor", [(32, -0.75), (97, -0.3), (384, 0.2), (510, 0.6), (1023, 1.0)])
@pytest.mark.parametrize("T1,T2", [(31, 11), (113, 203), (1023, 1024), (1, 239), (239, 1)])
def test_fused_l2_seqdiff(T1, T2, C, dfactor, dtype):
    from rgd_triton_amd import triton_fused_norm_func_fn, triton_norm_func_fn

    g = gen(2)
    C2 = max(1, int(C * (1 + dfactor)))
    x1, x2 = randn(g, 3, T1, C, dtype=dtype, scale=100.0), randn(g, 3, T2, C2, dtype=dtype, scale=100.0)
    d1, d2 = randn(g, 3, T1, C, dtype=dtype), randn(g, 3, T2, C2, dtype=dtype)
    x1g, x2g = to_gpu(x1, x2, requires_grad=True)
    y1, y2 = triton_fused_norm_func_fn(x1g, x2g, 1e-6)
    dx1, dx2 = torch.autograd.grad((y1, y2), (x1g, x2g), (d1.to("cuda"), d2.to("cuda")))
    assert_close(y1, oracle.l2_fwd(x1), dtype, name="y1")
    assert_close(y2, oracle.l2_fwd(x2), dtype, name="y2")
    assert_close_allow_inf(dx1, oracle.l2_bwd(d1, x1), dtype, name="dx1")
    assert_close_allow_inf(dx2, oracle.l2_bwd(d2, x2), dtype, name="dx2")
    if C == C2:
        assert torch.equal(y1, triton_norm_func_fn(x1g))


def test_fused_l2_module_and_determinism():
    from rgd_triton_amd import FusedL2Normalize2

    m = FusedL2Normalize2()
    g = gen(3)
    x1, x2 = randn(g, 60, 113, 257, dtype=torch.float16, scale=100.0), randn(g, 60, 31, 64, dtype=torch.float16)
    d1, d2 = randn(g, 60, 113, 257, dtype=torch.float16).cuda(), randn(g, 60, 31, 64, dtype=torch.float16).cuda()
    x1g, x2g = to_gpu(x1, x2, requires_grad=True)

    def step():
        y = m(x1g, x2g)
        return (*y, *torch.autograd.grad(y, (x1g, x2g), (d1, d2)))

    assert_repeats_bit_exact(step, ("y1", "y2", "dx1", "dx2"))
    assert m.cache.fwd is not None and m.cache.bwd is not None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [32, 63, 97, 122, 257, 384, 510, 740, 1023])
@pytest.mark.parametrize("T", [14, 128, 1024])
def test_l2_norm_race_condition(T, C, dtype):
    """The race test of tests/test_l2normalize.py: batch 60, its 9 widths, 250 repeats (three of its eight lengths)"""
    from rgd_triton_amd import triton_norm_func_fn

    g = gpu_gen(4)
    x = randn(g, 60, T, C, dtype=dtype)
    dy = randn(g, 60, T, C, dtype=dtype).cuda()
    xg = to_gpu(x, requires_grad=True)

    def step():
        y = triton_norm_func_fn(xg)
        return (y, *torch.autograd.grad(y, (xg,), dy))

    assert_repeats_bit_exact(step, ("y", "dx"))


FUSED_RACE_PAIRS = [(1, 239), (239, 1), (3, 799), (799, 3), (1024, 128), (97, 97), (128, 128), (200, 200), (256, 256),
                    (257, 257), (384, 384), (512, 512), (768, 768), (1024, 1024)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d,dfactor", [(32, -0.75), (63, 0.6), (97, -0.3), (122, 1.0), (257, 0.2), (257, -0.75), (384, -0.3),
                                       (510, 0.6), (740, 0.2), (1023, 1.0)])
@pytest.mark.parametrize("Tq,Tk", FUSED_RACE_PAIRS)
def test_fused_l2_norm_race_condition(Tq, Tk, d, dfactor, dtype):
    """The race test of tests/test_fused_l2normalize.py:283-354: batch 60, its 14 (Tq, Tk) pairs, 250 repeats of forward
    + backward; the widths follow its rule (dfactor < 0 narrows the first input, else the second).  Every one of its
    nine widths with one ratio (one width with two) instead of its full 9 x 5 grid."""
    from rgd_triton_amd import triton_fused_norm_func_fn

    CQ, CK = (int(-dfactor * d), d) if dfactor < 0 else (d, int(dfactor * d))
    torch.manual_seed(5)  # inputs made on the GPU: nothing here is compared with the CPU oracle
    B = 60
    qg, kg, gq, gk = (torch.randn(B, T, C, device="cuda", dtype=dtype) for T, C in ((Tq, CQ), (Tk, CK), (Tq, CQ), (Tk, CK)))
    qg.requires_grad_(True)
    kg.requires_grad_(True)

    def step():
        y = triton_fused_norm_func_fn(qg, kg)
        return (*y, *torch.autograd.grad(y, (qg, kg), (gq, gk)))

    assert_repeats_bit_exact(step, ("qo", "ko", "dq", "dk"))
