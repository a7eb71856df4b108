"""rgd_rms_bwd_noalloc: the RMSNorm backward for callers that cannot allocate.  Its partial dw rows live in a device
array inside the library instead of a caller's workspace; kernels and results are those of rgd_rms_bwd.  Called
through the C ABI, two calls in a row on the same GPU (the second on a smaller input, so it finds the first call's
contents in the shared array), each compared bit for bit with rgd_rms_bwd and against the CPU oracle."""
import pytest
import torch

from helpers import assert_close, gen, oracle, randn

pytestmark = pytest.mark.gpu


def _both(lib, hip, B, T, C, dtype, wdtype, shared, seed):
    g = gen(seed)
    x, dy = randn(g, B, T, C, dtype=dtype), randn(g, B, T, C, dtype=dtype)
    w = (1 + 0.1 * torch.randn((C,) if shared else (B, 1, C), generator=g)).to(wdtype)
    xg, dyg, wg = x.cuda(), dy.cuda(), w.cuda()
    code, wcode = hip.dtype_code(dtype), hip.dtype_code(wdtype)
    st = hip.stream_ptr(xg.device)
    t3 = hip.t3
    wsb = 0 if shared else wg.stride(0)
    out = {}
    for which in ("workspace", "noalloc"):
        dx = torch.full_like(xg, float("nan"))
        dw = torch.full_like(wg, float("nan"))
        dwsb = 0 if shared else dw.stride(0)
        if which == "workspace":
            n = lib.rgd_rms_bwd_workspace(B, T, C, 0, 0)
            ws = torch.empty(max(n, 16), dtype=torch.uint8, device="cuda")
            rc = lib.rgd_rms_bwd(B, T, C, t3(dyg), t3(xg), t3(wg, wsb), t3(dx), t3(dw, dwsb), int(shared), code, wcode,
                                 1e-6, ws.data_ptr(), n, st)
        else:
            # neither torch's allocator nor the device itself (an allocation made behind torch's back) gives up memory
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            rc = lib.rgd_rms_bwd_noalloc(B, T, C, t3(dyg), t3(xg), t3(wg, wsb), t3(dx), t3(dw, dwsb), int(shared), code,
                                         wcode, 1e-6, st)
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before
            assert torch.cuda.mem_get_info()[0] >= free_before
        assert rc == 0, lib.rgd_last_error()
        torch.cuda.synchronize()
        out[which] = (dx, dw)
    return out, oracle.rms_bwd(dy, x, w, 1e-6)


@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32),
                                          (torch.float16, torch.float32)])
def test_noalloc_matches_workspace_entry_point(dtype, wdtype):
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    assert lib.rgd_rms_bwd_noalloc_limit() == 16 << 20
    # first call: many blocks and partial rows; second: a smaller input with fewer and narrower rows, then a
    # per-batch weight, all through the same device array
    cases = [(4, 1024, 1536, True), (2, 37, 384, True), (3, 200, 1023, False), (1, 1, 32, True)]
    for i, (B, T, C, shared) in enumerate(cases):
        out, (dx_ref, dw_ref) = _both(lib, _hip, B, T, C, dtype, wdtype, shared, seed=40 + i)
        (dx_a, dw_a), (dx_b, dw_b) = out["workspace"], out["noalloc"]
        assert torch.equal(dx_a, dx_b) and torch.equal(dw_a, dw_b), (B, T, C, shared)
        assert not torch.isnan(dx_b.float()).any() and not torch.isnan(dw_b.float()).any()
        assert_close(dx_b, dx_ref, dtype, "rms", "dx")
        rows = B * T if shared else T
        assert_close(dw_b, dw_ref.to(dw_b.dtype), wdtype, "rms", "dw", atol_scale=3 * rows * C ** 0.5)


def test_noalloc_refuses_what_does_not_fit():
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    x = torch.zeros(2, 4, 65536, device="cuda")
    w = torch.ones(65536, device="cuda")
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    assert lib.rgd_rms_bwd_workspace(2, 4, 65536, 0, 0) > lib.rgd_rms_bwd_noalloc_limit()
    rc = lib.rgd_rms_bwd_noalloc(2, 4, 65536, _hip.t3(x), _hip.t3(x), _hip.t3(w, 0), _hip.t3(dx), _hip.t3(dw, 0), 1, 0, 0,
                                 1e-6, _hip.stream_ptr(x.device))
    assert rc == -4 and b"fixed scratch holds" in lib.rgd_last_error()
    torch.cuda.synchronize()
