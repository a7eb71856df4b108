"""Tile classes of a head-shared attention bias (rgd_attn_bias_classify and the kernels that read the classes): results
must equal those of the ordinary biased kernels (bit for bit for a dense bias, which those kernels still serve, and for an
all-zero one against a call without bias; to the last bits of the tensor type otherwise, because the bias enters the
logits before the product instead of after it), and the oracle within the reference's tolerance."""
import math

import pytest
import torch

from helpers import gen, oracle, randn

pytestmark = pytest.mark.gpu


def _mask(kind, B, Tq, Tk, g, dtype):
    """(B, 1, Tq, Tk) bias of the named kind, fp32 on the CPU"""
    NEG = float("-inf")
    m = torch.zeros(B, 1, Tq, Tk)
    if kind == "padding":  # a tenth of the last 256 keys hidden, per batch element
        span = min(256, Tk)
        for b in range(B):
            dead = Tk - span + torch.randperm(span, generator=g)[:max(span // 10, 1)]
            m[b, :, :, dead] = NEG
    elif kind == "blocks":  # documents packed into one sequence: block diagonal, block edges off the tile edges
        edges_q = sorted(set([0, Tq] + torch.randint(1, max(Tq, 2), (3,), generator=g).tolist()))
        for b in range(B):
            m[b] = NEG
            for a, e in zip(edges_q[:-1], edges_q[1:]):
                ka, ke = a * Tk // Tq, e * Tk // Tq
                m[b, :, a:e, ka:max(ke, ka + 1)] = 0
    elif kind == "random":  # 0 / -inf / finite tiles at random, tile by tile, key 0 visible to every row
        for b in range(B):
            for r in range(0, Tq, 32):
                for c in range(0, Tk, 64):
                    what = int(torch.randint(0, 4, (1,), generator=g))
                    if what == 1:
                        m[b, :, r:r + 32, c:c + 64] = NEG
                    elif what == 2:
                        m[b, :, r:r + 32, c:c + 64] = 0.5 * torch.randn(min(32, Tq - r), min(64, Tk - c), generator=g)
                    elif what == 3:
                        m[b, :, r:r + 32, c + int(torch.randint(0, 64, (1,), generator=g)) % max(Tk - c, 1)] = NEG
        m[:, :, :, 0] = 0
    elif kind == "dense":
        m = 0.5 * torch.randn(B, 1, Tq, Tk, generator=g)
    elif kind == "vpadding":  # the padding mask as a (B, 1, 1, Tk) vector
        return _mask("padding", B, Tq, Tk, g, dtype)[:, :, :1].contiguous()
    elif kind == "vdense":  # a finite value per key
        return 0.5 * torch.randn(B, 1, 1, Tk, generator=g)
    elif kind == "negzero":  # -0.0 is not +0.0 for the classes: such tiles must take the general path
        m = -m
    elif kind == "hidden_rows":  # some query rows see no key at all
        m[:, :, Tq // 3: Tq // 3 + 40, :] = NEG
    else:
        raise ValueError(kind)
    return m


CASES = [
    # kind, B, H, Tq, Tk, d, bias dtype (None: that of q), causal, shared by the batch
    ("padding", 2, 4, 512, 512, 64, None, False, False),
    ("padding", 2, 3, 300, 777, 64, None, False, False),
    ("padding", 1, 4, 1024, 640, 32, torch.float32, False, False),
    ("blocks", 2, 4, 640, 640, 64, None, False, False),
    ("blocks", 1, 2, 513, 450, 48, torch.float32, False, True),
    ("random", 2, 4, 384, 512, 64, None, False, False),
    ("random", 2, 2, 200, 2200, 64, None, False, True),
    ("random", 1, 4, 256, 256, 64, None, True, False),
    ("dense", 2, 4, 256, 320, 64, None, False, False),
    ("negzero", 1, 2, 128, 128, 64, None, False, False),
    ("hidden_rows", 1, 2, 256, 192, 64, None, False, False),
    ("padding", 2, 4, 4352 // 4, 4352 // 4, 64, None, False, False),
    ("vpadding", 2, 4, 512, 640, 64, None, False, False),
    ("vpadding", 2, 3, 300, 777, 32, torch.float32, False, False),
    ("vdense", 2, 4, 256, 320, 64, None, False, False),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(str(x).replace("torch.", "") for x in c))
def test_flash_attn_bias_classes(case, dtype):
    from rgd_triton_amd import _hip

    kind, B, H, Tq, Tk, d, bias_dtype, causal, shared_b = case
    lib = _hip.lib()
    g = gen(4242 + Tq + Tk)
    q, k, v, do = (randn(g, B, T, H, d, dtype=dtype) for T in (Tq, Tk, Tk, Tq))
    bias = _mask(kind, 1 if shared_b else B, Tq, Tk, g, dtype).to(bias_dtype or dtype)
    qg, kg, vg, dog = (x.cuda() for x in (q, k, v, do))
    # rows the 16-byte loads can read: a view into a buffer whose rows are padded to 16 elements
    tk_pad = (Tk + 15) // 16 * 16
    bg = torch.full((bias.shape[0], 1, bias.shape[2], tk_pad), float("nan"), dtype=bias.dtype, device="cuda")[..., :Tk]
    bg.copy_(bias)
    be = bg.expand(B, H, Tq, Tk)
    bdesc = _hip.Tensor4(be.data_ptr(), be.stride(0), be.stride(1), be.stride(2))
    bk = _hip.BIAS_VECTOR if bias.shape[2] == 1 else _hip.BIAS_MATRIX
    bd, code = _hip.dtype_code(bg.dtype), _hip.dtype_code(dtype)
    scale = 1.0 / math.sqrt(d)
    st = _hip.stream_ptr(qg.device)
    tqr = lib.rgd_attn_seqlen_q_rounded(Tq)
    delta_bytes = B * H * tqr * 4
    nbytes = lib.rgd_attn_bias_classes_bytes(B, H, Tq, Tk, d, bdesc, bk, bd)
    assert nbytes > 0
    classes = torch.empty(nbytes // 8, dtype=torch.int64, device="cuda")
    assert lib.rgd_attn_bias_classify(B, H, Tq, Tk, d, bdesc, bk, bd, classes.data_ptr(), nbytes, st) == 0, lib.rgd_last_error()
    fws = torch.empty(max(lib.rgd_attn_fwd_workspace(B, H, Tq, Tk, d), 16), dtype=torch.uint8, device="cuda")
    bws = torch.empty(lib.rgd_attn_bwd_workspace(B, H, Tq, Tk, d, 1), dtype=torch.uint8, device="cuda")

    def run(mode):
        """mode 0: no classes (a workspace too small for them), 1: the caller's classes, 2: classes the calls make"""
        o, dq = torch.empty_like(qg), torch.empty_like(qg)
        dk, dv = torch.empty_like(kg), torch.empty_like(kg)
        lse = torch.empty(B, H, tqr, dtype=torch.float32, device="cuda")
        t = {n: _hip.t4(x, False) for n, x in dict(q=qg, k=kg, v=vg, do=dog, o=o, dq=dq, dk=dk, dv=dv).items()}
        cp = classes.data_ptr() if mode == 1 else None
        # mode 1: delta and the bytes in which the two dK/dV launches agree on who serves a key block
        fb, bb = (fws.numel(), bws.numel()) if mode == 2 else (0, delta_bytes + (B * ((Tk + 127) // 128) + 32 if mode == 1 else 0))
        rc = lib.rgd_attn_fwd(B, H, Tq, Tk, d, t["q"], t["k"], t["v"], bdesc, bk, bd, t["o"], lse.data_ptr(), code, int(causal),
                              scale, cp, fws.data_ptr() if fb else None, fb, st)
        assert rc == 0, lib.rgd_last_error()
        rc = lib.rgd_attn_bwd(B, H, Tq, Tk, d, t["do"], t["q"], t["k"], t["v"], t["o"], lse.data_ptr(), bdesc, bk, bd, t["dq"],
                              t["dk"], t["dv"], None, code, int(causal), scale, 1, cp, bws.data_ptr(), bb, st)
        assert rc == 0, lib.rgd_last_error()
        torch.cuda.synchronize()
        return dict(o=o, lse=lse[:, :, :Tq], dq=dq, dk=dk, dv=dv)

    plain, given = run(0), run(1)
    # A bias that is mostly MIXED or COLUMN tiles (the dense ones) is handed to the ordinary kernels: the same bits.  Otherwise ZERO
    # tiles run the instructions of a tile without bias (the same bits again), NEG tiles are left out (they add exact
    # zeros), and on a MIXED or COLUMN tile (the -0.0 bias is all COLUMN tiles) the first product starts from the bias in
    # units of the raw scores (one rounding apart from adding it after the scaling), so results agree to rounding, not to
    # the bit.
    exact = kind in ("dense", "vdense")
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    for n in plain:
        a, b = plain[n], given[n]
        if exact:
            it = torch.int16 if a.element_size() == 2 else torch.int32
            assert torch.equal(a.view(it), b.view(it)), f"{n}: with classes != without ({(a.float() - b.float()).abs().max().item()})"
        elif n == "lse":
            torch.testing.assert_close(b, a, rtol=1e-5, atol=1e-5)
        else:
            big = a.float().abs().max().item()
            assert (a.float() - b.float()).abs().max().item() <= 2 * ulp * big, n
    # classes written by the calls themselves: items of a last round may be split here, so compare within tolerance
    own = run(2)
    for n in plain:
        torch.testing.assert_close(own[n].float(), plain[n].float(), rtol=2e-2, atol=2e-2, equal_nan=True)
    # and the oracle
    bfull = bias.expand(B, H, Tq, Tk)
    ref_o, ref_lse = oracle.attention_fwd(q, k, v, bfull, causal=causal)
    ref_dq, ref_dk, ref_dv = oracle.attention_bwd(do, q, k, v, bfull, causal=causal)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=4e-3, atol=4e-3)
    torch.testing.assert_close(given["o"].cpu().float(), ref_o.float(), **tol)
    torch.testing.assert_close(given["lse"].cpu(), ref_lse, rtol=1e-4, atol=1e-4)
    for n, ref in (("dq", ref_dq), ("dk", ref_dk), ("dv", ref_dv)):
        torch.testing.assert_close(given[n].cpu().float(), ref.float(), rtol=tol["rtol"], atol=tol["atol"] * max(1.0, ref.float().abs().max().item()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [32, 64])
def test_flash_attn_zero_bias_equals_no_bias(d, dtype):
    """A bias of +0.0 that the heads share runs, through its classes, the instructions of the kernels without bias:
    every output and gradient has the bits of a call without bias."""
    from rgd_triton_amd import flash_attn_func

    B, H, Tq, Tk = 2, 4, 640, 576
    g = gen(99 + d)
    q, k, v, do = (randn(g, B, T, H, d, dtype=dtype).cuda() for T in (Tq, Tk, Tk, Tq))
    bias = torch.zeros(B, 1, Tq, Tk, dtype=dtype, device="cuda")
    outs = []
    for bb in (None, bias):
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o, lse = flash_attn_func(qq, kk, vv, bb, return_lse=True)
        outs.append((o, lse) + torch.autograd.grad(o, (qq, kk, vv), do))
    for a, b, n in zip(outs[0], outs[1], ("o", "lse", "dq", "dk", "dv")):
        it = torch.int16 if a.element_size() == 2 else torch.int32
        assert torch.equal(a.view(it), b.view(it)), n


def test_flash_attn_shared_mask_classes_are_reused_and_follow_the_mask():
    """Through the Module API: the layers of a model that share one mask classify it once (the second call finds the
    classes of the first), an in-place change of the mask is seen (version counter), and forward + backward through
    autograd agree with the oracle either way."""
    from rgd_triton_amd import FlashAttention, clear_bias_classes_cache, functional

    g = gen(21)
    B, H, T, d, dtype = 2, 4, 320, 64, torch.bfloat16
    q, k, v, do = (randn(g, B, T, H, d, dtype=dtype) for _ in range(4))
    mask = torch.zeros(B, 1, T, T)
    mask[0, :, :, 250:] = float("-inf")
    mask[1, :, :, 300:] = float("-inf")
    mask = mask.to(dtype)
    attn = FlashAttention()
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    mg = mask.cuda()

    def run():
        o = attn(qg, kg, vg, bias=mg)
        return (o, *torch.autograd.grad(o, (qg, kg, vg), do.cuda()))

    def check(got, m):
        o_ref, _ = oracle.attention_fwd(q, k, v, m)
        g_ref = oracle.attention_bwd(do, q, k, v, m, False, None)
        for a, b in zip(got, (o_ref, *g_ref[:3])):
            assert (a.float().cpu() - b.float()).abs().max().item() < 3e-2

    clear_bias_classes_cache()
    first = run()
    entry = functional._classes_cache[mg.device]
    second = run()
    assert functional._classes_cache[mg.device][2] is entry[2]  # found, not written again
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    check(first, mask)
    # the mask changes in place: other keys are hidden now
    mg[:, :, :, 100:164] = float("-inf")
    mask2 = mg.cpu()
    third = run()
    assert functional._classes_cache[mg.device][2] is not entry[2]
    check(third, mask2)
    assert not torch.equal(third[0], first[0])
