"""The C-ABI entry points under HIP graph capture: the library launches only kernels, on the caller's
stream, and neither allocates nor synchronises, so a forward+backward sequence recorded once into a graph
must replay with the same results.  Every replay is checked bit for bit against an eager run on the same
inputs, with eager work and synchronisations between the replays and new input values on each replay."""
import ctypes
import math

import pytest
import torch

from helpers import gen, randn, oracle

pytestmark = pytest.mark.gpu


class _Sequence:
    """LN+RoPE, fused RMSNorm (two-launch backward) and attention with a bias (split tail round), forward and
    backward, writing into one of two sets of output buffers"""

    def __init__(self):
        from rgd_triton_amd import _hip

        self.hip, self.lib = _hip, _hip.lib()
        g, dt = gen(31), torch.bfloat16
        self.code = _hip.dtype_code(dt)
        B, T, H, D = 2, 700, 6, 64
        self.dims = (B, T, H, D)
        mk = lambda *s: randn(g, *s, dtype=dt).cuda()
        self.inp = dict(q=mk(B, T, H, D), k=mk(B, T, H, D), v=mk(B, T, H, D), g1=mk(B, T, H, D), g2=mk(B, T, H, D),
                        x1=mk(B, T, 384), x2=mk(B, 77, 640), d1=mk(B, T, 384), d2=mk(B, 77, 640),
                        w1=(1 + 0.1 * torch.randn(384, generator=g)).to(dt).cuda(),
                        w2=(1 + 0.1 * torch.randn(640, generator=g)).to(dt).cuda(),
                        bias=(0.3 * torch.randn(B, 1, T, T, generator=g)).to(dt).cuda())
        # the bias is shared by the heads, so the calls classify its tiles (inside the graph, when captured): batch
        # element 0 is a key mask, served by the kernels that read the classes; element 1 is dense, served by the others
        self.inp["bias"][0] = 0
        self.inp["bias"][0, :, :, T - 90::3] = float("-inf")
        self.pe = oracle.rotary_table(T + 1, 32, 10000.0, dt).cuda()
        lib = self.lib
        self.rms_ws = torch.empty(max(lib.rgd_rms_bwd_workspace(B, T, 384, 77, 640), 1), dtype=torch.uint8, device="cuda")
        self.attn_ws = torch.empty(lib.rgd_attn_bwd_workspace(B, H, T, T, D, 1), dtype=torch.uint8, device="cuda")
        self.attn_fws = torch.empty(max(lib.rgd_attn_fwd_workspace(B, H, T, T, D), 16), dtype=torch.uint8, device="cuda")
        self.lse = torch.empty(B, H, lib.rgd_attn_seqlen_q_rounded(T), dtype=torch.float32, device="cuda")

    def outputs(self):
        i = self.inp
        e = torch.empty_like
        return dict(qo=e(i["q"]), ko=e(i["k"]), dq_ln=e(i["q"]), dk_ln=e(i["k"]), y1=e(i["x1"]), y2=e(i["x2"]),
                    dx1=e(i["x1"]), dx2=e(i["x2"]), dw1=e(i["w1"]), dw2=e(i["w2"]), o=e(i["q"]), dq=e(i["q"]),
                    dk=e(i["q"]), dv=e(i["q"]))

    def run(self, out):
        hip, lib, i, code = self.hip, self.lib, self.inp, self.code
        B, T, H, D = self.dims
        st = hip.stream_ptr(torch.device("cuda"))
        t3, t4 = hip.t3, lambda t: hip.t4(t, False)
        pe = self.pe
        pe_args = (ctypes.c_void_p(pe.data_ptr()), pe.shape[1], pe.shape[2], pe.stride(0), pe.stride(1), code)
        rc = lib.rgd_ln_rope_qk_fwd(B, H, T, T, D, t4(i["q"]), t4(i["k"]), t4(out["qo"]), t4(out["ko"]), *pe_args, T, T,
                                    code, 1e-5, st)
        rc |= lib.rgd_ln_rope_qk_bwd(B, H, T, T, D, t4(i["q"]), t4(i["k"]), t4(i["g1"]), t4(i["g2"]), t4(out["dq_ln"]),
                                     t4(out["dk_ln"]), *pe_args, T, T, code, 1e-5, st)
        rc |= lib.rgd_fused_rms_fwd(B, T, 384, 77, 640, t3(i["x1"]), t3(i["w1"], 0), t3(out["y1"]), t3(i["x2"]),
                                    t3(i["w2"], 0), t3(out["y2"]), code, code, code, 1e-6, st)
        rc |= lib.rgd_fused_rms_bwd(B, T, 384, 77, 640, t3(i["d1"]), t3(i["x1"]), t3(i["w1"], 0), t3(out["dx1"]),
                                    t3(out["dw1"], 0), 1, t3(i["d2"]), t3(i["x2"]), t3(i["w2"], 0), t3(out["dx2"]),
                                    t3(out["dw2"], 0), 1, code, code, code, 1e-6, self.rms_ws.data_ptr(),
                                    self.rms_ws.numel(), st)
        be = i["bias"].expand(B, H, T, T)
        bdesc = hip.Tensor4(be.data_ptr(), be.stride(0), be.stride(1), be.stride(2))
        scale = 1.0 / math.sqrt(D)
        # attention consumes the LN+RoPE outputs of this same sequence
        rc |= lib.rgd_attn_fwd(B, H, T, T, D, t4(out["qo"]), t4(out["ko"]), t4(i["v"]), bdesc, hip.BIAS_MATRIX, code,
                               t4(out["o"]), self.lse.data_ptr(), code, 0, scale, None, self.attn_fws.data_ptr(),
                               self.attn_fws.numel(), st)
        rc |= lib.rgd_attn_bwd(B, H, T, T, D, t4(i["g1"]), t4(out["qo"]), t4(out["ko"]), t4(i["v"]), t4(out["o"]),
                               self.lse.data_ptr(), bdesc, hip.BIAS_MATRIX, code, t4(out["dq"]), t4(out["dk"]),
                               t4(out["dv"]), None, code, 0, scale, 1, None, self.attn_ws.data_ptr(), self.attn_ws.numel(), st)
        assert rc == 0, lib.rgd_last_error()


def test_c_abi_sequence_replays_from_a_graph():
    seq = _Sequence()
    eager_out, graph_out = seq.outputs(), seq.outputs()
    seq.run(eager_out)  # also creates each kernel's one-time launch attributes outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        seq.run(graph_out)
    for rep in range(4):
        for t in graph_out.values():
            t.fill_(float("nan"))
        for name in ("q", "x1", "v", "d2"):  # new values in the graph's input buffers (eager kernels)
            seq.inp[name].mul_(-0.75 if rep % 2 else 1.25)
        seq.inp["bias"].copy_(seq.inp["bias"].flip(0))  # mask and dense bias change places: other classes on replay
        torch.cuda.synchronize()
        seq.run(eager_out)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, t in graph_out.items():
            assert not torch.isnan(t.float()).any(), f"replay {rep}: {name} holds NaN"
            assert torch.equal(t, eager_out[name]), f"replay {rep}: {name} differs from the eager run"


@pytest.mark.skip(reason="recording an autograd backward into a HIP graph aborted inside the runtime's end-of-capture "
                         "call when it was first tried; no output of that run was kept and reading the code has not "
                         "shown a cause, so the case stays off the GPU and the package refuses it with an error "
                         "(functional._no_capture)")
def test_autograd_forward_backward_replays_from_a_graph():
    """What the case would be: the Module API, forward and backward through autograd, recorded and replayed."""
    from rgd_triton_amd import FlashAttention

    g = gen(32)
    q, k, v, do = (randn(g, 2, 300, 4, 64, dtype=torch.bfloat16).cuda() for _ in range(4))
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    attn = FlashAttention()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):  # warm-up off the default stream, as torch's graph recipe asks
        torch.autograd.grad(attn(q, k, v), (q, k, v), do)
    torch.cuda.current_stream().wait_stream(side)
    eager = torch.autograd.grad(attn(q, k, v), (q, k, v), do)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = torch.autograd.grad(attn(q, k, v), (q, k, v), do)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(captured, eager):
            assert torch.equal(a, b)
