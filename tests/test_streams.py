"""Calls on side streams: every operator launches on torch's current stream and takes its scratch per call from the
caching allocator (which never hands a block to another stream while it is in use), so two streams that run different
problems at the same time give, bit for bit, what each gives alone on the default stream."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DT = torch.bfloat16


def _problem(seed, T, C, Ta, H, D):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(DT).cuda()
    return dict(x=mk(2, T, C), w=(1 + 0.1 * torch.randn(C, generator=g)).to(DT).cuda(), dy=mk(2, T, C),
                q=mk(2, Ta, H, D), k=mk(2, Ta, H, D), v=mk(2, Ta, H, D), do=mk(2, Ta, H, D),
                bias=mk(2, 1, Ta, Ta))


def _run(p):
    from rgd_triton_amd import flash_attn_func, triton_fused_ln_func_fn, triton_rms_func_fn

    x, w = p["x"].clone().requires_grad_(True), p["w"].clone().requires_grad_(True)
    y = triton_rms_func_fn(x, w, 1e-6)
    dx, dw = torch.autograd.grad(y, (x, w), p["dy"])
    q, k, v = (p[n].clone().requires_grad_(True) for n in "qkv")
    qn, kn = triton_fused_ln_func_fn(q, k, False)
    o = flash_attn_func(qn, kn, v, p["bias"])
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), p["do"])
    return [y, dx, dw, o, dq, dk, dv]


def test_two_streams_match_default_stream():
    pa, pb = _problem(1, 700, 1536, 520, 4, 64), _problem(2, 333, 4096, 390, 3, 128)
    ref_a, ref_b = _run(pa), _run(pb)
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    for _ in range(6):  # interleaved enqueues: the two streams overlap on the GPU
        with torch.cuda.stream(sa):
            outs_a.append(_run(pa))
        with torch.cuda.stream(sb):
            outs_b.append(_run(pb))
    torch.cuda.synchronize()
    for outs, ref in ((outs_a, ref_a), (outs_b, ref_b)):
        for got in outs:
            for a, r in zip(got, ref):
                assert torch.equal(a, r)


def test_two_host_threads():
    """two host threads, each on its own stream, call the operators at the same time (autograd adds its own worker
    thread for the backward passes): results equal the single-threaded ones bit for bit"""
    import threading

    pa, pb = _problem(3, 257, 768, 200, 2, 64), _problem(4, 129, 2048, 333, 3, 32)
    ref = {"a": _run(pa), "b": _run(pb)}
    torch.cuda.synchronize()
    outs, errors = {"a": [], "b": []}, []

    def work(name, prob):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(8):
                    outs[name].append(_run(prob))
            stream.synchronize()
        except Exception as e:  # surfaced in the main thread below
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=work, args=("a", pa)), threading.Thread(target=work, args=("b", pb))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for name in ("a", "b"):
        assert len(outs[name]) == 8
        for got in outs[name]:
            for a, r in zip(got, ref[name]):
                assert torch.equal(a, r)
