"""GPU parity of FusedRMSNorm / triton_rms_func_fn against the CPU oracle.
Counterpart of the reference's tests/test_rms.py (parity :126-184, race :188-246)."""
import pytest
import torch

from helpers import DTYPES, assert_close, assert_repeats_bit_exact, gen, gpu_gen, oracle, randn, to_gpu

pytestmark = pytest.mark.gpu


def _run(B, T, C, dtype, unique_bw, wdtype=None, seed=0, eps=1e-6):
    from rgd_triton_amd import triton_rms_func_fn

    wdtype = wdtype or dtype
    g = gen(seed)
    x = randn(g, B, T, C, dtype=dtype)
    w = (1 + 0.1 * torch.randn((B, 1, C) if unique_bw else (C,), generator=g)).to(wdtype)
    dy = randn(g, B, T, C, dtype=dtype)
    xg, wg = to_gpu(x, w, requires_grad=True)
    y = triton_rms_func_fn(xg, wg, eps)
    dx, dw = torch.autograd.grad(y, (xg, wg), dy.to("cuda"))
    y_ref = oracle.rms_fwd(x, w, eps)
    dx_ref, dw_ref = oracle.rms_bwd(dy, x, w, eps)
    return (y, dx, dw), (y_ref, dx_ref, dw_ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [32, 63, 97, 122, 257, 384, 510, 740, 1023, 1024, 1536, 2048, 4096])
@pytest.mark.parametrize("unique_bw", [False, True])
@pytest.mark.parametrize("T", [14, 128, 1024])
def test_rms_norm(T, unique_bw, C, dtype):
    B = 4
    (y, dx, dw), (y_ref, dx_ref, dw_ref) = _run(B, T, C, dtype, unique_bw)
    assert_close(y, y_ref, dtype, "rms", "y")
    assert_close(dx, dx_ref, dtype, "rms", "dx")
    # the reference widens atol for dw by 3*rows*sqrt(C) (tests/test_rms.py:182-184)
    rows = T if unique_bw else B * T
    assert_close(dw, dw_ref, dtype, "rms", "dw", atol_scale=3 * rows * C ** 0.5)
    assert dw.shape == dw_ref.shape and dw.dtype == dw_ref.dtype


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [2049, 3072, 5120, 6144, 8192])
@pytest.mark.parametrize("unique_bw", [False, True])
@pytest.mark.parametrize("T", [7, 300])
def test_rms_norm_wide_rows(T, unique_bw, C, dtype):
    """Rows wider than one wavefront keeps in registers: four wavefronts share a row.  Odd C takes the
    unvectorised loads, whose limit is 4096 elements."""
    B = 2
    (y, dx, dw), (y_ref, dx_ref, dw_ref) = _run(B, T, C, dtype, unique_bw, seed=C + T)
    assert_close(y, y_ref, dtype, "rms", "y")
    assert_close(dx, dx_ref, dtype, "rms", "dx")
    rows = T if unique_bw else B * T
    assert_close(dw, dw_ref, dtype, "rms", "dw", atol_scale=3 * rows * C ** 0.5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,unique_bw", [(8200, False), (10001, False), (12288, True), (16384, False), (20000, False),
                                         (20001, True), (32768, True), (65536, False), (70003, False)])
def test_rms_norm_streamed_rows(C, unique_bw, dtype):
    """Rows beyond the register-resident limit take the two-pass streaming kernel, at any width like the reference
    (it loops over channel blocks, rmsnorm_cached.py:198-219): the dw sums of the backward stay in registers one
    slab of 16384 channels (8192 on the unaligned path) at a time."""
    B, T = 2, 37
    (y, dx, dw), (y_ref, dx_ref, dw_ref) = _run(B, T, C, dtype, unique_bw, seed=C)
    assert_close(y, y_ref, dtype, "rms", "y")
    assert_close(dx, dx_ref, dtype, "rms", "dx")
    rows = T if unique_bw else B * T
    assert_close(dw, dw_ref, dtype, "rms", "dw", atol_scale=3 * rows * C ** 0.5)


@pytest.mark.parametrize("T", [1, 3, 31, 97, 200, 1025])
def test_rms_ragged_rows(T):
    (y, dx, dw), (y_ref, dx_ref, dw_ref) = _run(3, T, 384, torch.bfloat16, False)
    assert_close(y, y_ref, torch.bfloat16, "rms", "y")
    assert_close(dx, dx_ref, torch.bfloat16, "rms", "dx")
    assert_close(dw, dw_ref, torch.bfloat16, "rms", "dw", atol_scale=3 * 3 * T * 384 ** 0.5)


@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                          (torch.float32, torch.bfloat16)])
def test_rms_mixed_weight_dtype(dtype, wdtype):
    (y, dx, dw), (y_ref, dx_ref, dw_ref) = _run(2, 130, 768, dtype, False, wdtype=wdtype)
    assert dw.dtype == wdtype
    assert_close(y, y_ref, dtype, "rms", "y")
    assert_close(dx, dx_ref, dtype, "rms", "dx")
    assert_close(dw, dw_ref, wdtype, "rms", "dw", atol_scale=3 * 260 * 768 ** 0.5)


def test_rms_config1_fp32_tight():
    """Benchmark configuration 1: (4,1024,1024) fp32, w = 1 + 0.1 N(0,1), eps 1e-6; fp32 bar <= 1e-5 relative."""
    (y, dx, dw), (y_ref, dx_ref, dw_ref) = _run(4, 1024, 1024, torch.float32, False, seed=1001)
    for a, r, n in ((y, y_ref, "y"), (dx, dx_ref, "dx"), (dw, dw_ref, "dw")):
        err = (a.cpu() - r).abs().max() / r.abs().max()
        assert err <= 1e-5, f"{n}: relative error {err:.3e}"


def test_rms_strided_views():
    """x and dy that are slices of a wider buffer (row stride != C) and a weight of shape (1,1,C)."""
    from rgd_triton_amd import triton_rms_func_fn

    g = gen(5)
    big = randn(g, 2, 50, 3 * 256, dtype=torch.float16)
    w = (1 + 0.1 * torch.randn(1, 1, 256, generator=g)).to(torch.float16)
    dyb = randn(g, 2, 50, 2 * 256, dtype=torch.float16)
    x = big[:, :, 256:512]
    dy = dyb[:, :, 256:]
    bg, wg = to_gpu(big, w, requires_grad=True)
    xg = bg[:, :, 256:512]
    y = triton_rms_func_fn(xg, wg, 1e-6)
    dbig, dw = torch.autograd.grad(y, (bg, wg), dyb.to("cuda")[:, :, 256:])
    dx_ref, dw_ref = oracle.rms_bwd(dy, x, w)
    assert_close(y, oracle.rms_fwd(x, w), torch.float16, "rms", "y")
    assert_close(dbig[:, :, 256:512], dx_ref, torch.float16, "rms", "dx")
    assert dw.shape == (1, 1, 256)
    assert_close(dw, dw_ref, torch.float16, "rms", "dw", atol_scale=3 * 100 * 16)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("unique_bw", [True, False])
@pytest.mark.parametrize("C", [32, 63, 97, 122, 257, 384, 510, 740, 1023])
@pytest.mark.parametrize("T", [14, 31, 97, 128, 200, 384, 768, 1024])
def test_rms_norm_race_condition(T, C, unique_bw, dtype):
    """The reference's race test at its own strength (tests/test_rms.py:187-246): batch 60, its 9 widths x 8 lengths x
    both weight forms x 3 dtypes, 250 repeats.  The reference allows dx and dw to move by rounding noise; here y, dx
    and dw must reproduce bit for bit."""
    _race(60, T, C, dtype, unique_bw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,T", [(1536, 512), (6144, 67), (12288, 19), (40000, 5)])
def test_rms_deterministic_wide(C, T, dtype):
    """the same loop on the multi-wavefront and streaming kernels (widths the reference's tests do not reach)"""
    _race(60 if C < 40000 else 12, T, C, dtype, False)


def _race(B, T, C, dtype, unique_bw):
    from rgd_triton_amd import triton_rms_func_fn

    g = gpu_gen(7)
    x = randn(g, B, T, C, dtype=dtype, shift=0.5)
    w = randn(g, *((B, 1, C) if unique_bw else (C,)), dtype=dtype, scale=0.1, shift=1.0)
    dy = randn(g, B, T, C, dtype=dtype)
    xg, wg = to_gpu(x, w, requires_grad=True)
    dyg = dy.to("cuda")

    def step():
        y = triton_rms_func_fn(xg, wg, 1e-6)
        return (y, *torch.autograd.grad(y, (xg, wg), dyg))

    assert_repeats_bit_exact(step, ("y", "dx", "dw"))


def test_module_state_dict_and_cache():
    from rgd_triton_amd import FusedRMSNorm

    m = FusedRMSNorm(256, eps=1e-5, device="cuda", dtype=torch.float32)
    assert list(m.state_dict().keys()) == ["weight"] and torch.all(m.weight == 1)
    assert m.cache.fwd is None and m.cache.bwd is None and m.cache.bwd_dw is None
    x = torch.randn(2, 7, 256, device="cuda", requires_grad=True)
    y = m(x)
    y.sum().backward()
    assert m.cache.fwd is not None and m.cache.bwd is not None
    assert_close(y, oracle.rms_fwd(x.detach().cpu(), m.weight.detach().cpu(), 1e-5), torch.float32, "rms", "y")
    m.enable_cache(False)
    assert m.cache is None
    y2 = m(x)
    assert torch.equal(y, y2)
    m2 = FusedRMSNorm(256, elementwise_affine=False)
    assert m2.weight is None
    with pytest.raises(AssertionError, match="Must pass in a weight tensor"):
        m2(x)
    with pytest.raises(AssertionError, match="only supports int dims"):
        FusedRMSNorm((256,))
