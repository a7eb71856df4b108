"""GPU parity of FusedHeadLayerNorm, RoPE and FusedLNRoPE.  Counterparts of the reference's
tests/test_head_layernorm.py, tests/test_head_rope.py and tests/test_fused_ln_rope.py."""
import pytest
import torch

from helpers import DTYPES, assert_close, assert_repeats_bit_exact, gen, gpu_gen, oracle, randn, to_gpu

pytestmark = pytest.mark.gpu

SEQ_PAIRS = [(31, 11), (23, 138), (113, 203), (128, 217), (108, 256), (256, 512), (1023, 1024), (1, 239), (239, 1)]
D_R = [(32, 32), (64, 32), (64, 64), (128, 32), (128, 64), (128, 96), (128, 128)]


def _qk(g, B, H, Tq, Tk, D, dtype, heads_second, shift=0.0, scale=1.0):
    if heads_second:
        return randn(g, B, H, Tq, D, dtype=dtype, shift=shift, scale=scale), randn(g, B, H, Tk, D, dtype=dtype, shift=shift, scale=scale)
    return randn(g, B, Tq, H, D, dtype=dtype, shift=shift, scale=scale), randn(g, B, Tk, H, D, dtype=dtype, shift=shift, scale=scale)


# ---------------------------------------------------------------- head LayerNorm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("D", [32, 64, 96, 128, 256, 40, 59])
@pytest.mark.parametrize("Tq,Tk", [(14, 14), (200, 200), (113, 203), (1, 239), (1024, 1023)])
def test_head_ln(Tq, Tk, D, heads_second, dtype):
    from rgd_triton_amd import triton_fused_ln_func_fn

    g = gen(0)
    q, k = _qk(g, 4, 9, Tq, Tk, D, dtype, heads_second, shift=0.5, scale=2.0)
    dq_o, dk_o = _qk(g, 4, 9, Tq, Tk, D, dtype, heads_second)
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo, ko = triton_fused_ln_func_fn(qg, kg, heads_second, 1e-6)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (dq_o.to("cuda"), dk_o.to("cuda")))
    assert_close(qo, oracle.head_ln_fwd(q), dtype, name="qo")
    assert_close(ko, oracle.head_ln_fwd(k), dtype, name="ko")
    assert_close(dq, oracle.head_ln_bwd(dq_o, q), dtype, name="dq")
    assert_close(dk, oracle.head_ln_bwd(dk_o, k), dtype, name="dk")


def test_head_ln_layout_invariance_and_views():
    """op(x.transpose(1,2), heads_second=True) == op(x, heads_second=False).transpose(1,2), bit for bit;
    q, k taken as views of a packed qkv buffer (token stride 3*h*d)."""
    from rgd_triton_amd import FusedHeadLayerNorm

    g = gen(1)
    qkv = randn(g, 2, 77, 3, 6, 64, dtype=torch.bfloat16).to("cuda")
    q, k, _ = qkv.unbind(2)  # (B,T,H,D) views, token stride 3*H*D
    m = FusedHeadLayerNorm()
    a_q, a_k = m(q, k, heads_second=False)
    b_q, b_k = m(q.transpose(1, 2), k.transpose(1, 2), heads_second=True)
    assert torch.equal(a_q, b_q.transpose(1, 2)) and torch.equal(a_k, b_k.transpose(1, 2))
    assert_close(a_q, oracle.head_ln_fwd(q.cpu()), torch.bfloat16, name="q view")
    c_q, _ = m(q.contiguous(), k.contiguous(), heads_second=False)
    assert torch.equal(a_q, c_q)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("which", ["ln", "rope", "ln_rope"])
def test_head_ops_compact_addressing_equals_general(which, heads_second, dtype):
    """Tensors whose rows lie at one distance (contiguous ones) take kernels that address them with a base and a 32-bit
    offset; any other layout takes the general kernels.  The same values through both, forward and backward, must give
    the same bits: here contiguous tensors against views into buffers with one spare head between the tokens."""
    from rgd_triton_amd import triton_fused_ln_func_fn, triton_fused_ln_rope_fn, triton_rope_fn

    g = gen(31)
    B, H, Tq, Tk, D, R = 3, 5, 150, 97, 64, 32
    q, k = _qk(g, B, H, Tq, Tk, D, dtype, heads_second, shift=0.3, scale=1.5)
    gq, gk = _qk(g, B, H, Tq, Tk, D, dtype, heads_second)
    pe = oracle.rotary_table(max(Tq, Tk) + 1, R, dtype=dtype).to("cuda")
    cut = (Tq * 3 // 4, Tk)

    def spread(t):
        """the same values as a view with a spare head (heads_second: a spare token) between the rows of a token"""
        t = t.cuda()
        big = torch.full((t.shape[0], t.shape[1], t.shape[2] + 1, t.shape[3]), float("nan"), dtype=t.dtype, device="cuda")
        view = big[:, :, : t.shape[2]]
        view.copy_(t)
        return view

    def run(a, b, ga, gb):
        a, b = a.detach().requires_grad_(True), b.detach().requires_grad_(True)
        if which == "ln":
            out = triton_fused_ln_func_fn(a, b, heads_second, 1e-6)
        elif which == "rope":
            out = triton_rope_fn(a, b, pe, cut, heads_second)
        else:
            out = triton_fused_ln_rope_fn(a, b, pe, cut, heads_second)
        return (*out, *torch.autograd.grad(out, (a, b), (ga, gb)))

    dense = run(q.cuda(), k.cuda(), gq.cuda(), gk.cuda())
    spaced = run(spread(q), spread(k), spread(gq), spread(gk))
    for a, b, n in zip(dense, spaced, ("qo", "ko", "dq", "dk")):
        assert not torch.isnan(b.float()).any(), n
        assert torch.equal(a, b), n


# ---------------------------------------------------------------- RoPE
def _table(P, R, dtype, axial=False):
    if axial:
        L = int(P ** 0.5) + 1
        return oracle.axial_rotary_table(L, R, 32.0, dtype)
    return oracle.rotary_table(P, R, 10000.0, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,R", D_R)
@pytest.mark.parametrize("cut", [0, 0.5, 0.75, 1.0])
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("T", [14, 97, 384])
def test_rope(T, heads_second, cut, D, R, dtype):
    from rgd_triton_amd import triton_rope_fn

    g = gen(0)
    q, k = _qk(g, 4, 9, T, T, D, dtype, heads_second)
    gq, gk = _qk(g, 4, 9, T, T, D, dtype, heads_second)
    pe = _table(T + 1, R, dtype, axial=True)[:, : T + 1].contiguous()
    cutoff = (int(cut * T), int(cut * T))
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo, ko = triton_rope_fn(qg, kg, pe.to("cuda"), seq_cutoff=cutoff, heads_second=heads_second)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    qr, kr = oracle.rope_fwd(q, k, pe, cutoff, heads_second)
    dqr, dkr = oracle.rope_bwd(gq, gk, pe, cutoff, heads_second)
    for a, r, n in ((qo, qr, "qo"), (ko, kr, "ko"), (dq, dqr, "dq"), (dk, dkr, "dk")):
        assert_close(a, r, dtype, "rope", n)
    if cut == 0:
        assert torch.equal(qo, qg) and torch.equal(dk.cpu(), gk)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("Tq,Tk", SEQ_PAIRS)
def test_rope_seqdiff(Tq, Tk, heads_second, dtype):
    from rgd_triton_amd import RoPE

    g = gen(2)
    D, R = 128, 96
    q, k = _qk(g, 3, 5, Tq, Tk, D, dtype, heads_second)
    gq, gk = _qk(g, 3, 5, Tq, Tk, D, dtype, heads_second)
    pe = _table(max(Tq, Tk) + 3, R, torch.float32)  # fp32 table with 16-bit q/k is allowed
    cutoff = (int(0.75 * Tq), int(0.5 * Tk))
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo, ko = RoPE()(qg, kg, pe.to("cuda"), seq_cutoff=cutoff, heads_second=heads_second)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    qr, kr = oracle.rope_fwd(q, k, pe, cutoff, heads_second)
    dqr, dkr = oracle.rope_bwd(gq, gk, pe, cutoff, heads_second)
    for a, r, n in ((qo, qr, "qo"), (ko, kr, "ko"), (dq, dqr, "dq"), (dk, dkr, "dk")):
        assert_close(a, r, dtype, "rope", n)
    assert not torch.equal(qo, qg) or cutoff[0] == 0  # out of place: the input is untouched
    assert torch.equal(qg.detach().cpu(), q)


def test_rope_errors_and_cutoff_forms():
    from rgd_triton_amd import triton_rope_fn

    q = torch.randn(1, 2, 16, 64, device="cuda")
    pe = oracle.rotary_table(16, 32).to("cuda")
    with pytest.raises(AssertionError):  # the reference requires T < P strictly
        triton_rope_fn(q, q, pe)
    pe = oracle.rotary_table(17, 32).to("cuda")
    a = triton_rope_fn(q, q, pe, seq_cutoff=None)
    b = triton_rope_fn(q, q, pe, seq_cutoff=16)
    c = triton_rope_fn(q, q, pe, seq_cutoff=[16, 16])
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], c[1])
    big = torch.randn(1, 2, 16, 160, device="cuda")
    with pytest.raises(AssertionError, match="up to 128"):
        triton_rope_fn(big, big, pe)
    pe.requires_grad_(True)
    qq = q.clone().requires_grad_(True)
    out = triton_rope_fn(qq, qq, pe)
    with pytest.raises(AssertionError, match="does not support gradients in position embeddings"):
        torch.autograd.grad(out[0].sum(), (qq, pe))


# ---------------------------------------------------------------- LayerNorm + RoPE
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,R", D_R)
@pytest.mark.parametrize("cut", [0, 0.5, 1.0])
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("T", [31, 200])
def test_ln_rope(T, heads_second, cut, D, R, dtype):
    from rgd_triton_amd import triton_fused_ln_rope_fn

    g = gen(0)
    q, k = _qk(g, 4, 9, T, T, D, dtype, heads_second, shift=0.3, scale=1.5)
    gq, gk = _qk(g, 4, 9, T, T, D, dtype, heads_second)
    pe = _table(T + 1, R, dtype, axial=True)[:, : T + 1].contiguous()
    cutoff = (int(cut * T), int(cut * T))
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo, ko = triton_fused_ln_rope_fn(qg, kg, pe.to("cuda"), seq_cutoff=cutoff, heads_second=heads_second, norm_eps=1e-6)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    qr, kr = oracle.ln_rope_fwd(q, k, pe, cutoff, heads_second, 1e-6)
    dqr, dkr = oracle.ln_rope_bwd(gq, gk, q, k, pe, cutoff, heads_second, 1e-6)
    for a, r, n in ((qo, qr, "qo"), (ko, kr, "ko"), (dq, dqr, "dq"), (dk, dkr, "dk")):
        assert_close(a, r, dtype, "ln_rope", n)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("Tq,Tk", SEQ_PAIRS)
def test_ln_rope_seqdiff(Tq, Tk, heads_second, dtype):
    from rgd_triton_amd import FusedLNRoPE

    g = gen(4)
    D, R = 64, 32
    q, k = _qk(g, 3, 5, Tq, Tk, D, dtype, heads_second, shift=-0.2, scale=3.0)
    gq, gk = _qk(g, 3, 5, Tq, Tk, D, dtype, heads_second)
    pe = _table(max(Tq, Tk) + 1, R, dtype)
    cutoff = (int(0.75 * Tq), Tk)
    qg, kg = to_gpu(q, k, requires_grad=True)
    qo, ko = FusedLNRoPE()(qg, kg, pe.to("cuda"), seq_cutoff=cutoff, heads_second=heads_second, eps=1e-5)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    qr, kr = oracle.ln_rope_fwd(q, k, pe, cutoff, heads_second, 1e-5)
    dqr, dkr = oracle.ln_rope_bwd(gq, gk, q, k, pe, cutoff, heads_second, 1e-5)
    for a, r, n in ((qo, qr, "qo"), (ko, kr, "ko"), (dq, dqr, "dq"), (dk, dkr, "dk")):
        assert_close(a, r, dtype, "ln_rope", n)


def test_ln_rope_equals_ln_then_rope_fp32():
    """fusion: FusedLNRoPE == RoPE(FusedHeadLayerNorm) in fp32 within fp32 tolerance"""
    from rgd_triton_amd import triton_fused_ln_func_fn, triton_fused_ln_rope_fn, triton_rope_fn

    g = gen(5)
    q, k = _qk(g, 2, 4, 100, 60, 96, torch.float32, False)
    pe = oracle.rotary_table(101, 64).to("cuda")
    qg, kg = to_gpu(q, k)
    a = triton_fused_ln_rope_fn(qg, kg, pe, heads_second=False)
    b = triton_rope_fn(*triton_fused_ln_func_fn(qg, kg, False), pe, heads_second=False)
    assert_close(a[0], b[0], torch.float32, name="q")
    assert_close(a[1], b[1], torch.float32, name="k")


def test_ln_rope_config2_slice():
    """Benchmark configuration 2 at reduced batch: q,k (2,2048,16,64) bf16, heads_second=False, eps 1e-5,
    R=32, theta 10000, cutoff (2048,2048), P = 2049."""
    from rgd_triton_amd import FusedLNRoPE

    g = gen(1002)
    q, k = _qk(g, 2, 16, 2048, 2048, 64, torch.bfloat16, False)
    gq, gk = _qk(g, 2, 16, 2048, 2048, 64, torch.bfloat16, False)
    pe = oracle.rotary_table(2049, 32, 10000.0, torch.bfloat16)
    qg, kg = to_gpu(q, k, requires_grad=True)
    m = FusedLNRoPE()
    qo, ko = m(qg, kg, pe.to("cuda"), seq_cutoff=(2048, 2048), heads_second=False, eps=1e-5)
    dq, dk = torch.autograd.grad((qo, ko), (qg, kg), (gq.to("cuda"), gk.to("cuda")))
    qr, kr = oracle.ln_rope_fwd(q, k, pe, (2048, 2048), False, 1e-5)
    dqr, dkr = oracle.ln_rope_bwd(gq, gk, q, k, pe, (2048, 2048), False, 1e-5)
    for a, r, n in ((qo, qr, "qo"), (ko, kr, "ko"), (dq, dqr, "dq"), (dk, dkr, "dk")):
        assert_close(a, r, torch.bfloat16, "ln_rope", n)


RACE_PAIRS = [(1, 239), (239, 1), (3, 799), (799, 3), (1024, 128), (97, 97), (128, 128), (200, 200), (256, 256),
              (257, 257), (384, 384), (512, 512), (768, 768), (1024, 1024)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("Tq,Tk", RACE_PAIRS)
def test_head_ln_race_condition(Tq, Tk, D, heads_second, dtype):
    """The reference's race test at its own strength (tests/test_head_layernorm.py:214-): batch 60, 4 heads, 250 repeats"""
    from rgd_triton_amd import triton_fused_ln_func_fn

    g = gpu_gen(6)
    q, k = _qk(g, 60, 4, Tq, Tk, D, dtype, heads_second)
    gq, gk = (t.cuda() for t in _qk(g, 60, 4, Tq, Tk, D, dtype, heads_second))
    qg, kg = to_gpu(q, k, requires_grad=True)

    def step():
        out = triton_fused_ln_func_fn(qg, kg, heads_second)
        return (*out, *torch.autograd.grad(out, (qg, kg), (gq, gk)))

    assert_repeats_bit_exact(step, ("qo", "ko", "dq", "dk"))


@pytest.mark.parametrize("which", ["rope", "ln_rope"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("heads_second", [True, False])
@pytest.mark.parametrize("D,R", [(32, 32), (64, 32), (128, 96), (128, 128)])
@pytest.mark.parametrize("Tq,Tk", RACE_PAIRS)
def test_rope_race_condition(Tq, Tk, D, R, heads_second, dtype, which):
    """The race tests of tests/test_head_rope.py and tests/test_fused_ln_rope.py: batch 60, their 14 length pairs, 250
    repeats, on four of their seven (head dim, rotary dim) combinations; cutoffs inside both sequences."""
    from rgd_triton_amd import triton_fused_ln_rope_fn, triton_rope_fn

    g = gpu_gen(6)
    q, k = _qk(g, 60, 4, Tq, Tk, D, dtype, heads_second)
    gq, gk = (t.cuda() for t in _qk(g, 60, 4, Tq, Tk, D, dtype, heads_second))
    pe = oracle.rotary_table(max(Tq, Tk) + 1, R, dtype=dtype).to("cuda")
    qg, kg = to_gpu(q, k, requires_grad=True)
    cut = (max(1, Tq * 3 // 4), max(1, Tk * 2 // 3))
    fn = (lambda: triton_rope_fn(qg, kg, pe, cut, heads_second)) if which == "rope" else \
        (lambda: triton_fused_ln_rope_fn(qg, kg, pe, cut, heads_second))

    def step():
        out = fn()
        return (*out, *torch.autograd.grad(out, (qg, kg), (gq, gk)))

    assert_repeats_bit_exact(step, ("qo", "ko", "dq", "dk"))
