#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-extra] [--skip-cpu]

Headline workload (BASELINE.json configs[1]): FusedLNRoPE forward+backward on q and k, each
(8,2048,16,64) bf16, heads_second=False, LayerNorm eps 1e-5 without affine, rotary theta 10000 on the
first 32 channels of the first 2048 tokens.  One step = one forward launch + one backward launch
through the C ABI (the two calls the autograd Function makes), on inputs resident in HBM.  Four
independent buffer sets (4 x 268 MB) are used in rotation so that no step finds its inputs in the
256 MB Infinity Cache left there by the previous step.

Prints ONE JSON line: value = algorithmic GB/s of the whole step, `roofline` for the dominant
kernel (the backward) from HIP events recorded around every launch inside the timed region,
(minus the measured cost of an event), `cpu_baseline` = the CPU oracle timed on this host on a bounded sample, and `extra` with the other
benchmark configurations (attention TFLOP/s, RMSNorm2 / head LayerNorm GB/s) and the Module-API timing.
"""
import argparse
import ctypes
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16
BWD_KERNELS = "attn_bwd_dq_kernel + attn_bwd_dkv_kernel (one rgd_attn_bwd call)"

PROFILE_SUMMARY = os.path.join("profiles", "head_rows_lnrope_config2.md")


def profile_figures(path=PROFILE_SUMMARY):
    """Figures of the dominant kernel that only a profiler run can give (HBM traffic counters, the kernel-trace
    duration), read from the committed rocprofv3 summary: lines `bench.<key> = <value>` at its end, next to the
    commit they were measured at.  Nothing is reported when the file or a key is missing."""
    out = {}
    try:
        for line in open(os.path.join(ROOT, path)):
            if line.startswith("bench.") and "=" in line:
                k, v = line[len("bench."):].split("=", 1)
                out[k.strip()] = v.strip()
    except OSError:
        pass
    return out


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=1000,
                    help="untimed steps; the GPU needs tens of milliseconds of work to reach its steady clocks")
    ap.add_argument("--skip-extra", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--only", default="", help="run only this extra workload (for profiling)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch 5 plain 256 MiB device copies (reads 256 MiB, writes 256 MiB each) so that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings can be scaled to bytes")
    return ap.parse_args()


def event_ms(pairs):
    return [a.elapsed_time(b) for a, b in pairs]


def timed_loop(torch, step_fns, steps, warmup):
    """step_fns: list of callables (one per buffer set), each returns nothing and launches
    [fwd, bwd] given an event recorder.  Returns (wall ms per step, event span ms per step, fwd ms list,
    bwd ms list, event-to-event gap ms)."""
    n = len(step_fns)
    # untimed: bring the clocks to their steady state whatever --warmup says, then the W warm-up steps
    spin_up(torch, lambda i: step_fns[i % n](None), 0.1)
    for i in range(warmup):
        step_fns[i % n](None)
    # timed region: exactly `steps` steps between two synchronisations; only the two bracketing events
    # are on the stream, so the launches run back to back
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        step_fns[i % n](None)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    gpu_span = e0.elapsed_time(e1) / steps
    # the same steps again with an event after every launch: per-kernel durations for the roofline
    # (an event between two launches costs a few microseconds of stream time, which is why this is a
    # separate pass and not the one `value` comes from).  A fourth event recorded straight after the third
    # measures that cost (event to event with nothing between); it is subtracted from both intervals.
    # (the events are created beforehand: creating them inside the loop costs the host more per step than the GPU
    # needs for it, and an interval then includes the wait for the host)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    for i, rec in enumerate(evs):
        step_fns[(i + steps) % n](rec)
        rec[3].record()
    torch.cuda.synchronize()
    gap = statistics.median(e[2].elapsed_time(e[3]) for e in evs)
    fwd = [e[0].elapsed_time(e[1]) - gap for e in evs]
    bwd = [e[1].elapsed_time(e[2]) - gap for e in evs]
    return wall, gpu_span, fwd, bwd, gap


def make_ln_rope_sets(torch, nsets, B=8, T=2048, H=16, D=64, R=32, seed=1002):
    import rgd_oracle as oracle

    g = torch.Generator().manual_seed(seed)
    pe = oracle.rotary_table(T + 1, R, 10000.0, torch.bfloat16).cuda()
    sets = []
    for _ in range(nsets):
        t = [torch.randn(B, T, H, D, generator=g).to(torch.bfloat16).cuda() for _ in range(4)]  # q k gq gk
        outs = [torch.empty_like(t[0]) for _ in range(4)]  # qo ko dq dk
        sets.append((t, outs))
    return pe, sets


def ln_rope_steps(torch, pe, sets, eps=1e-5):
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    fns = []
    for (q, k, gq, gk), (qo, ko, dq, dk) in sets:
        B, T, H, D = q.shape
        pe_args = (ctypes.c_void_p(pe.data_ptr()), pe.shape[1], pe.shape[2], pe.stride(0), pe.stride(1), _hip.RGD_BF16)
        d = {n: _hip.t4(x, False) for n, x in dict(q=q, k=k, gq=gq, gk=gk, qo=qo, ko=ko, dq=dq, dk=dk).items()}
        stream = _hip.stream_ptr(q.device)

        def step(rec, d=d, B=B, T=T, H=H, D=D, pe_args=pe_args, stream=stream):
            if rec:
                rec[0].record()
            rc = lib.rgd_ln_rope_qk_fwd(B, H, T, T, D, d["q"], d["k"], d["qo"], d["ko"], *pe_args, T, T, _hip.RGD_BF16,
                                        eps, stream)
            if rec:
                rec[1].record()
            rc |= lib.rgd_ln_rope_qk_bwd(B, H, T, T, D, d["q"], d["k"], d["gq"], d["gk"], d["dq"], d["dk"], *pe_args, T, T,
                                         _hip.RGD_BF16, eps, stream)
            if rec:
                rec[2].record()
            assert rc == 0, lib.rgd_last_error()

        fns.append(step)
    return fns


def cpu_baseline_ln_rope(torch, B=8, T=2048, H=16, D=64, R=32, reps=3):
    """The CPU oracle (oracle/rgd_oracle.py, PyTorch eager fp32) on the full workload, all host threads."""
    import rgd_oracle as oracle

    g = torch.Generator().manual_seed(1002)
    q, k, gq, gk = (torch.randn(B, T, H, D, generator=g).to(torch.bfloat16) for _ in range(4))
    pe = oracle.rotary_table(T + 1, R, 10000.0, torch.bfloat16)
    times = []
    for i in range(reps + 1):
        t0 = time.perf_counter()
        oracle.ln_rope_fwd(q, k, pe, (T, T), False, 1e-5)
        oracle.ln_rope_bwd(gq, gk, q, k, pe, (T, T), False, 1e-5)
        if i:
            times.append(time.perf_counter() - t0)
    nbytes = 5 * 2 * B * T * H * D * 2
    return {"value": round(nbytes / statistics.median(times) / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"oracle ln_rope_fwd+ln_rope_bwd on q,k ({B},{T},{H},{D}) bf16, median of {reps}",
            "host_cpus": os.cpu_count()}


def torch_eager_ln_rope(torch, B=8, T=2048, H=16, D=64, R=32, iters=20):
    """The headline step written with PyTorch's own GPU operators (F.layer_norm in fp32, the rotation as slices and a
    stack, autograd for the backward) on the same shapes: what a user has on this GPU without fused kernels.  A second
    reported baseline, not a target."""
    import torch.nn.functional as F

    try:
        g = torch.Generator().manual_seed(1002)
        q, k, gq, gk = (torch.randn(B, T, H, D, generator=g).to(torch.bfloat16).cuda() for _ in range(4))
        q.requires_grad_(True)
        k.requires_grad_(True)
        inv = 10000.0 ** (-torch.arange(0, R, 2, dtype=torch.float32) / R)
        ang = torch.arange(T, dtype=torch.float32)[:, None] * inv[None, :]
        sin = ang.sin().repeat_interleave(2, dim=-1)[None, :, None, :].cuda()
        cos = ang.cos().repeat_interleave(2, dim=-1)[None, :, None, :].cuda()

        def one(x):
            y = F.layer_norm(x.float(), (D,), eps=1e-5)
            r, rest = y[..., :R], y[..., R:]
            rot = torch.stack((-r[..., 1::2], r[..., 0::2]), dim=-1).flatten(-2)
            return torch.cat((r * cos + rot * sin, rest), dim=-1).to(x.dtype)

        def step(_=None):
            qo, ko = one(q), one(k)
            torch.autograd.grad((qo, ko), (q, k), (gq, gk))

        spin_up(torch, step, 0.05)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / iters
        nbytes = 5 * 2 * B * T * H * D * 2
        return {"value": round(nbytes / ms / 1e6, 1), "unit": "GB/s", "ms_per_step": round(ms, 4),
                "what": f"torch {torch.__version__} eager operators + autograd on the same GPU, same algorithmic bytes"}
    except Exception as e:
        return {"error": f"{type(e).__name__}: {str(e)[:100]}"}


# ------------------------------------------------------------------------------------------------
# extra workloads (reported under "extra", not the headline value)
# ------------------------------------------------------------------------------------------------

def _cpu_time(fn, reps=2):
    times = []
    for i in range(reps + 1):
        t0 = time.perf_counter()
        fn()
        if i:
            times.append(time.perf_counter() - t0)
    return statistics.median(times)


def cpu_extra(torch, kind, **kw):
    """The CPU oracle on a bounded sample of an extra workload (a few seconds each), timed beside the GPU figure."""
    import rgd_oracle as oracle

    g = torch.Generator().manual_seed(7)
    cores = torch.get_num_threads()
    if kind == "rms":
        B, shapes, dtype = kw["B"], kw["shapes"], kw["dtype"]
        xs = [torch.randn(B, T, C, generator=g).to(dtype) for T, C in shapes]
        ds = [torch.randn(B, T, C, generator=g).to(dtype) for T, C in shapes]
        ws = [(1 + 0.1 * torch.randn(C, generator=g)).to(dtype) for _, C in shapes]

        def run():
            for x, d, w in zip(xs, ds, ws):
                oracle.rms_fwd(x, w)
                oracle.rms_bwd(d, x, w)
        t = _cpu_time(run)
        nbytes = 5 * sum(x.numel() * x.element_size() for x in xs)
        return {"value": round(nbytes / t / 1e9, 3), "unit": "GB/s", "ms": round(t * 1e3, 2), "cores": cores, "kind": "port",
                "sample": "oracle rms_fwd+rms_bwd on the full workload"}
    if kind == "head_ln":
        B, T, H, D, dtype = kw["B"], kw["T"], kw["H"], kw["D"], kw["dtype"]
        q, k, gq, gk = (torch.randn(1, T, H, D, generator=g).to(dtype) for _ in range(4))

        def run():
            for x, d in ((q, gq), (k, gk)):
                oracle.head_ln_fwd(x)
                oracle.head_ln_bwd(d, x)
        t = _cpu_time(run)
        nbytes = 5 * 2 * q.numel() * q.element_size()
        return {"value": round(nbytes / t / 1e9, 3), "unit": "GB/s", "ms": round(t * 1e3, 2), "cores": cores, "kind": "port",
                "sample": f"oracle head_ln_fwd+head_ln_bwd on one of {B} batch elements"}
    if kind == "attention":
        B, T, H, D, dtype, bias = kw["B"], kw["T"], kw["H"], kw["D"], kw["dtype"], kw["bias"]
        hs = 2  # two heads of one batch element: T*T*2 fp32 scores at a time
        q, k, v, do = (torch.randn(1, T, hs, D, generator=g).to(dtype) for _ in range(4))
        bs = None if bias is None else bias[:1, :hs if bias.shape[1] > 1 else 1].cpu()

        def run():
            oracle.attention_fwd(q, k, v, bs)
            oracle.attention_bwd(do, q, k, v, bs)
        t = _cpu_time(run, reps=1)
        flops = 14.0 * hs * T * T * D
        return {"value": round(flops / t / 1e12, 4), "unit": "TFLOP/s", "ms": round(t * 1e3, 1), "cores": cores, "kind": "port",
                "sample": f"oracle attention_fwd+attention_bwd on 2 of {B * H} (batch, head) pairs"}
    raise ValueError(kind)

def spin_up(torch, fn, seconds=0.06):
    """Untimed launches for `seconds`: after an idle spell (allocation, input generation on the host) the GPU
    needs tens of milliseconds of work before its clocks reach their steady state, and a kernel timed during
    that ramp reads 5-20 % slow."""
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn(i)
            i += 1
        torch.cuda.synchronize()


def time_api(torch, fn, iters=30, warmup=5):
    spin_up(torch, lambda i: fn())
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def attention_case(torch, name, B, T, H, D, dtype, bias_kind, iters=20, with_cpu=False, causal=False):
    """fwd+bwd through the C ABI with events around the forward and the backward call"""
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    g = torch.Generator().manual_seed(1003)
    q, k, v, do = (torch.randn(B, T, H, D, generator=g).to(dtype).cuda() for _ in range(4))
    bias = None
    if bias_kind == "full":
        bias = (0.5 * torch.randn(B, H, T, T, generator=g)).to(dtype)
        i = torch.arange(T)
        bias.masked_fill_((i[None, :] // 128) > (i[:, None] // 128), float("-inf"))
        bias = bias.cuda()
    elif bias_kind == "broadcast":
        bias = torch.zeros(B, 1, T, T)
        for b in range(B):
            dead = T - 256 + torch.randperm(256, generator=g)[:26]
            bias[b, :, :, dead] = float("-inf")
        bias = bias.to(dtype).cuda()
    elif bias_kind in ("vector", "mask_full"):  # config 5's key mask as a (B,1,1,T) vector / written out for every head
        bias = torch.zeros(B, 1, 1, T)
        for b in range(B):
            dead = T - 256 + torch.randperm(256, generator=g)[:26]
            bias[b, :, :, dead] = float("-inf")
        bias = bias.to(dtype).cuda()
        if bias_kind == "mask_full":
            bias = bias.expand(B, H, T, T).contiguous()
    elif bias_kind == "zero_shared":  # comparison workloads (--only): what the bias of config 5 costs
        bias = torch.zeros(B, 1, T, T, dtype=dtype, device="cuda")
    elif bias_kind == "dense_shared":
        bias = (0.5 * torch.randn(B, 1, T, T, generator=g)).to(dtype).cuda()
    elif bias_kind == "dense_full":
        bias = (0.5 * torch.randn(B, H, T, T, generator=g)).to(dtype).cuda()
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    tqr = lib.rgd_attn_seqlen_q_rounded(T)
    lse = torch.empty(B, H, tqr, dtype=torch.float32, device="cuda")
    mode = {"auto": 0, "two_kernel": 1, "one_pass": 2}[os.environ.get("RGD_ATTN_BWD", "auto")]
    ws = torch.empty(lib.rgd_attn_bwd_workspace(B, H, T, T, D, mode), dtype=torch.uint8, device="cuda")
    fws = torch.empty(max(lib.rgd_attn_fwd_workspace(B, H, T, T, D), 16), dtype=torch.uint8, device="cuda")
    code = _hip.dtype_code(dtype)
    if bias is None:
        bdesc, bk, bd = _hip.Tensor4(None, 0, 0, 0), _hip.BIAS_NONE, _hip.RGD_F32
    else:
        be = bias.expand(B, H, T, T)
        bdesc = _hip.Tensor4(be.data_ptr(), be.stride(0), be.stride(1), be.stride(2))
        bk, bd = (_hip.BIAS_VECTOR if bias.shape[2] == 1 else _hip.BIAS_MATRIX), code
    t = {n: _hip.t4(x, False) for n, x in dict(q=q, k=k, v=v, do=do, o=o, dq=dq, dk=dk, dv=dv).items()}
    st = _hip.stream_ptr(q.device)
    scale = 1.0 / math.sqrt(D)
    # tile classes of a head-shared bias: written once per step, in the forward (as the autograd Function does), and
    # passed to both calls; RGD_BENCH_CLASSES=0 passes none and lets each call classify on its own
    cls_bytes = lib.rgd_attn_bias_classes_bytes(B, H, T, T, D, bdesc, bk, bd) if bias is not None else 0
    if os.environ.get("RGD_BENCH_CLASSES", "1") == "0":
        cls_bytes = 0
    cls_buf = torch.empty(max(cls_bytes, 8) // 8, dtype=torch.int64, device="cuda")
    cls_ptr = cls_buf.data_ptr() if cls_bytes else None

    def fwd(classify=True):
        if cls_bytes and classify:
            assert lib.rgd_attn_bias_classify(B, H, T, T, D, bdesc, bk, bd, cls_ptr, cls_bytes, st) == 0, lib.rgd_last_error()
        assert lib.rgd_attn_fwd(B, H, T, T, D, t["q"], t["k"], t["v"], bdesc, bk, bd, t["o"], lse.data_ptr(), code, int(causal),
                                scale, cls_ptr, fws.data_ptr(), fws.numel(), st) == 0, lib.rgd_last_error()

    def bwd():
        assert lib.rgd_attn_bwd(B, H, T, T, D, t["do"], t["q"], t["k"], t["v"], t["o"], lse.data_ptr(), bdesc, bk, bd,
                                t["dq"], t["dk"], t["dv"], None, code, int(causal), scale, mode, cls_ptr, ws.data_ptr(), ws.numel(), st) == 0, \
            lib.rgd_last_error()

    # forward and backward alternate as in a training step; the clocks are brought to their steady state first
    def step(_):
        fwd()
        bwd()

    spin_up(torch, step, 0.1)
    evs = []
    for _ in range(iters):
        e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e[0].record()
        fwd()
        e[1].record()
        bwd()
        e[2].record()
        evs.append(e)
    torch.cuda.synchronize()
    f_ms = statistics.mean(e[0].elapsed_time(e[1]) for e in evs)
    b_ms = statistics.mean(e[1].elapsed_time(e[2]) for e in evs)
    # the forward when the classes of the bias are already there (a model whose layers share one mask classifies it once
    # for all of them): reported beside fwd_ms, which includes the classification
    f_shared = None
    if cls_bytes:
        pairs = []
        for _ in range(iters):
            a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fwd(classify=False)
            b_.record()
            bwd()
            pairs.append((a, b_))
        torch.cuda.synchronize()
        f_shared = round(statistics.mean(event_ms(pairs)), 4)
    # causal: the pairs above the diagonal do not exist, so half of the dense count is credited
    flops = 14.0 * B * H * T * T * D * (0.5 if causal else 1.0)
    tot = f_ms + b_ms
    cpu = cpu_extra(torch, "attention", B=B, T=T, H=H, D=D, dtype=dtype, bias=bias) if with_cpu and not causal else None
    sdpa = torch_sdpa_case(torch, q, k, v, do, bias, flops) if with_cpu and not causal else None
    # roofline of the slower of the two calls (MFMA-bound; algorithmic FLOPs 4/14 forward, 10/14 backward)
    f_tf, b_tf = flops * 4 / 14 / f_ms / 1e9, flops * 10 / 14 / b_ms / 1e9
    slow_bwd = b_tf <= f_tf
    roof = {"bound": "mfma", "kernel": BWD_KERNELS if slow_bwd else "attn_fwd_kernel (rgd_attn_fwd)",
            "achieved": round(b_tf if slow_bwd else f_tf, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round((b_tf if slow_bwd else f_tf) / MFMA_PEAK_TFLOPS, 4),
            "avg_launch_ms": round(b_ms if slow_bwd else f_ms, 4),
            "duration_source": "HIP events around the call, mean of %d" % iters}
    return {"workload": name, "roofline": roof, "cpu_baseline": cpu, "torch_sdpa": sdpa, "bias_bytes": None if bias is None else bias.numel() * bias.element_size(), "fwd_ms": round(f_ms, 4), "bwd_ms": round(b_ms, 4), "fwd_ms_classes_given": f_shared,
            "tflops": round(flops / tot / 1e9, 2), "fwd_tflops": round(flops * 4 / 14 / f_ms / 1e9, 2),
            "bwd_tflops": round(flops * 10 / 14 / b_ms / 1e9, 2), "frac_mfma_peak": round(flops / tot / 1e9 / MFMA_PEAK_TFLOPS, 4)}


def torch_sdpa_case(torch, q, k, v, do, bias, flops, iters=10):
    """PyTorch's own fused attention (scaled_dot_product_attention, whatever backend it picks on this GPU) on the same
    tensors, forward + backward through autograd: a second reported baseline next to the CPU one, not a target."""
    import torch.nn.functional as F

    try:
        ql, kl, vl = (t.detach().transpose(1, 2).requires_grad_(True) for t in (q, k, v))  # (B,h,T,d) views
        dot = do.transpose(1, 2)

        def step(_=None):
            o = F.scaled_dot_product_attention(ql, kl, vl, attn_mask=bias)
            torch.autograd.grad(o, (ql, kl, vl), dot)

        spin_up(torch, step, 0.05)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / iters
        return {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2), "what": f"torch {torch.__version__} F.scaled_dot_product_attention fwd+bwd, default backend"}
    except Exception as e:  # no kernel for this shape / dtype on this build
        return {"error": f"{type(e).__name__}: {str(e)[:100]}"}


def time_pair(torch, fwd, bwd, nsets, iters=60, warmup=8):
    """average ms of fwd(i) and of bwd(i) (i = buffer set), each timed as a run of back-to-back launches"""
    out = []
    for fn in (fwd, bwd):
        spin_up(torch, lambda i: fn(i % nsets))
        for i in range(warmup):
            fn(i % nsets)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(iters):
            fn(i % nsets)
        b.record()
        torch.cuda.synchronize()
        out.append(a.elapsed_time(b) / iters)
    return out


def rows_result(torch, name, fwd, bwd, fwd_bytes, bwd_bytes, nsets, api=None):
    """HBM-bound operator through the C ABI on rotating buffer sets (algorithmic bytes: every tensor read or
    written once); `api` optionally times the same step through the Module API + autograd."""
    f_ms, b_ms = time_pair(torch, fwd, bwd, nsets)
    tot = f_ms + b_ms
    r = {"workload": name, "fwd_us": round(f_ms * 1e3, 2), "bwd_us": round(b_ms * 1e3, 2),
         "fwd_gbs": round(fwd_bytes / f_ms / 1e6, 1), "bwd_gbs": round(bwd_bytes / b_ms / 1e6, 1),
         "gbs": round((fwd_bytes + bwd_bytes) / tot / 1e6, 1),
         "frac_hbm_peak": round((fwd_bytes + bwd_bytes) / tot / 1e6 / HBM_PEAK_GBS, 4), "path": "C ABI, back-to-back launches"}
    # warm figure: one buffer set over and over, so whatever fits stays in the 256 MB Infinity Cache
    wf_ms, wb_ms = time_pair(torch, fwd, bwd, 1)
    r["warm_fwd_us"], r["warm_bwd_us"] = round(wf_ms * 1e3, 2), round(wb_ms * 1e3, 2)
    r["warm_gbs"] = round((fwd_bytes + bwd_bytes) / (wf_ms + wb_ms) / 1e6, 1)
    if api is not None:
        r["module_api_ms"] = round(time_api(torch, api, 30, 5), 4)
    return r


def rms_case(torch, name, B, shapes, dtype, nsets, with_api=True, with_cpu=False):
    """FusedRMSNorm (one shape) or FusedRMSNorm2 (two shapes) forward+backward, shared (C,) weights"""
    import rgd_triton_amd as rgd
    from rgd_triton_amd import _hip

    lib, t3 = _hip.lib(), _hip.t3
    code = _hip.dtype_code(dtype)
    es = torch.empty(0, dtype=dtype).element_size()
    st = _hip.stream_ptr(torch.device("cuda"))
    (T1, C1), (T2, C2) = shapes[0], (shapes[1] if len(shapes) > 1 else (0, 0))
    mk = lambda T, C: [torch.randn(B, T, C, device="cuda").to(dtype) for _ in range(nsets)]
    x1, d1, x2, d2 = mk(T1, C1), mk(T1, C1), mk(T2, max(C2, 1)), mk(T2, max(C2, 1))
    y1, y2 = [torch.empty_like(t) for t in x1], [torch.empty_like(t) for t in x2]
    w1 = (1 + 0.1 * torch.randn(C1, device="cuda")).to(dtype)
    w2 = (1 + 0.1 * torch.randn(max(C2, 1), device="cuda")).to(dtype)
    dw1, dw2 = torch.empty_like(w1), torch.empty_like(w2)
    ws = lib.rgd_rms_bwd_workspace(B, T1, C1, T2, C2)
    wbuf = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda")
    if T2 == 0:
        def fwd(i):
            assert lib.rgd_rms_fwd(B, T1, C1, t3(x1[i]), t3(w1, 0), t3(y1[i]), code, code, 1e-6, st) == 0, lib.rgd_last_error()

        def bwd(i):
            assert lib.rgd_rms_bwd(B, T1, C1, t3(d1[i]), t3(x1[i]), t3(w1, 0), t3(y1[i]), t3(dw1, 0), 1, code, code, 1e-6,
                                   wbuf.data_ptr(), ws, st) == 0, lib.rgd_last_error()
    else:
        def fwd(i):
            assert lib.rgd_fused_rms_fwd(B, T1, C1, T2, C2, t3(x1[i]), t3(w1, 0), t3(y1[i]), t3(x2[i]), t3(w2, 0), t3(y2[i]),
                                         code, code, code, 1e-6, st) == 0, lib.rgd_last_error()

        def bwd(i):
            assert lib.rgd_fused_rms_bwd(B, T1, C1, T2, C2, t3(d1[i]), t3(x1[i]), t3(w1, 0), t3(y1[i]), t3(dw1, 0), 1,
                                         t3(d2[i]), t3(x2[i]), t3(w2, 0), t3(y2[i]), t3(dw2, 0), 1, code, code, code, 1e-6,
                                         wbuf.data_ptr(), ws, st) == 0, lib.rgd_last_error()
    n = B * (T1 * C1 + T2 * C2) * es
    api = None
    if with_api:
        xa = x1[0].clone().requires_grad_(True)
        if T2 == 0:
            m = rgd.FusedRMSNorm(C1, device="cuda", dtype=dtype)
            api = lambda: torch.autograd.grad(m(xa), (xa, m.weight), d1[0])
        else:
            xb = x2[0].clone().requires_grad_(True)
            m = rgd.FusedRMSNorm2((C1, C2), device="cuda", dtype=dtype)
            api = lambda: torch.autograd.grad(m(xa, xb), (xa, xb, m.weight1, m.weight2), (d1[0], d2[0]))
    r = rows_result(torch, name, fwd, bwd, 2 * n, 3 * n, nsets, api)
    r["cpu_baseline"] = cpu_extra(torch, "rms", B=B, shapes=shapes, dtype=dtype) if with_cpu else None
    return r


def head_ln_case(torch, name, B, T, H, D, dtype, nsets, with_cpu=False):
    import rgd_triton_amd as rgd
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    code = _hip.dtype_code(dtype)
    st = _hip.stream_ptr(torch.device("cuda"))
    mk = lambda: [torch.randn(B, T, H, D, device="cuda").to(dtype) for _ in range(nsets)]
    q, k, gq, gk = mk(), mk(), mk(), mk()
    qo, ko = [torch.empty_like(t) for t in q], [torch.empty_like(t) for t in k]
    d = [{n: _hip.t4(x[i], False) for n, x in dict(q=q, k=k, gq=gq, gk=gk, qo=qo, ko=ko).items()} for i in range(nsets)]

    def fwd(i):
        assert lib.rgd_ln_qk_fwd(B, H, T, T, D, d[i]["q"], d[i]["k"], d[i]["qo"], d[i]["ko"], code, 1e-6, st) == 0, \
            lib.rgd_last_error()

    def bwd(i):
        assert lib.rgd_ln_qk_bwd(B, H, T, T, D, d[i]["q"], d[i]["k"], d[i]["gq"], d[i]["gk"], d[i]["qo"], d[i]["ko"], code,
                                 1e-6, st) == 0, lib.rgd_last_error()

    qa, ka = q[0].clone().requires_grad_(True), k[0].clone().requires_grad_(True)
    m = rgd.FusedHeadLayerNorm()
    api = lambda: torch.autograd.grad(m(qa, ka, heads_second=False), (qa, ka), (gq[0], gk[0]))
    n = 2 * B * T * H * D * torch.empty(0, dtype=dtype).element_size()
    r = rows_result(torch, name, fwd, bwd, 2 * n, 3 * n, nsets, api)
    r["cpu_baseline"] = cpu_extra(torch, "head_ln", B=B, T=T, H=H, D=D, dtype=dtype) if with_cpu else None
    return r


def rope_case(torch, name, B, T, H, D, R, dtype, nsets):
    """RoPE alone (rgd_rope_qk forward, then with the rotation sign flipped: its backward) on q and k"""
    import rgd_oracle as oracle
    from rgd_triton_amd import _hip

    lib = _hip.lib()
    code = _hip.dtype_code(dtype)
    st = _hip.stream_ptr(torch.device("cuda"))
    pe = oracle.rotary_table(T + 1, R, 10000.0, dtype).cuda()
    pe_args = (ctypes.c_void_p(pe.data_ptr()), pe.shape[1], pe.shape[2], pe.stride(0), pe.stride(1), code)
    mk = lambda: [torch.randn(B, T, H, D, device="cuda").to(dtype) for _ in range(nsets)]
    q, k, gq, gk = mk(), mk(), mk(), mk()
    qo, ko = [torch.empty_like(t) for t in q], [torch.empty_like(t) for t in k]
    d = [{n: _hip.t4(x[i], False) for n, x in dict(q=q, k=k, gq=gq, gk=gk, qo=qo, ko=ko).items()} for i in range(nsets)]

    def fwd(i):
        assert lib.rgd_rope_qk(B, H, T, T, D, d[i]["q"], d[i]["k"], d[i]["qo"], d[i]["ko"], *pe_args, T, T, 0, code, st) == 0, \
            lib.rgd_last_error()

    def bwd(i):
        assert lib.rgd_rope_qk(B, H, T, T, D, d[i]["gq"], d[i]["gk"], d[i]["qo"], d[i]["ko"], *pe_args, T, T, 1, code, st) == 0, \
            lib.rgd_last_error()

    n = 2 * B * T * H * D * torch.empty(0, dtype=dtype).element_size()
    return rows_result(torch, name, fwd, bwd, 2 * n, 2 * n, nsets)  # the backward reads dy and writes dx: two passes


def l2_case(torch, name, B, shapes, dtype, nsets):
    """FusedL2Normalize2 forward+backward through the C ABI"""
    from rgd_triton_amd import _hip

    lib, t3 = _hip.lib(), _hip.t3
    code = _hip.dtype_code(dtype)
    es = torch.empty(0, dtype=dtype).element_size()
    st = _hip.stream_ptr(torch.device("cuda"))
    (T1, C1), (T2, C2) = shapes
    mk = lambda T, C: [torch.randn(B, T, C, device="cuda").to(dtype) for _ in range(nsets)]
    x1, d1, x2, d2 = mk(T1, C1), mk(T1, C1), mk(T2, C2), mk(T2, C2)
    y1, y2 = [torch.empty_like(t) for t in x1], [torch.empty_like(t) for t in x2]

    def fwd(i):
        assert lib.rgd_fused_l2_fwd(B, T1, C1, T2, C2, t3(x1[i]), t3(y1[i]), t3(x2[i]), t3(y2[i]), code, 1e-6, st) == 0, \
            lib.rgd_last_error()

    def bwd(i):
        assert lib.rgd_fused_l2_bwd(B, T1, C1, T2, C2, t3(d1[i]), t3(x1[i]), t3(y1[i]), t3(d2[i]), t3(x2[i]), t3(y2[i]), code, 1e-6,
                                    st) == 0, lib.rgd_last_error()

    n = B * (T1 * C1 + T2 * C2) * es
    return rows_result(torch, name, fwd, bwd, 2 * n, 3 * n, nsets)


def extras(torch, only="", with_cpu=False):
    import rgd_triton_amd as rgd

    out = []
    bf = torch.bfloat16

    def want(n):
        return not only or only == n

    if want("attn_c3"):
        out.append(attention_case(torch, "attn_c3: (4,4096,16,64) bf16 no bias", 4, 4096, 16, 64, bf, None, with_cpu=with_cpu))
    if want("attn_c4"):
        out.append(attention_case(torch, "attn_c4: (2,2048,16,128) fp16 full bias", 2, 2048, 16, 128, torch.float16, "full", with_cpu=with_cpu))
    if want("attn_c5"):
        out.append(attention_case(torch, "attn_c5: (2,4352,24,64) bf16 broadcast bias", 2, 4352, 24, 64, bf, "broadcast", with_cpu=with_cpu))

    # comparison workloads, only when named: the config-5 shape without bias, with an all-zero and with a dense head-shared
    # bias; the config-4 shape with a finite bias (no -inf blocks to leave out)
    if only == "attn_c5_nobias":
        out.append(attention_case(torch, "attn_c5_nobias: (2,4352,24,64) bf16 no bias", 2, 4352, 24, 64, bf, None))
    if only == "attn_c5_zero":
        out.append(attention_case(torch, "attn_c5_zero: (2,4352,24,64) bf16 (B,1,T,T) bias of zeros", 2, 4352, 24, 64, bf, "zero_shared"))
    if only == "attn_c5_dense":
        out.append(attention_case(torch, "attn_c5_dense: (2,4352,24,64) bf16 (B,1,T,T) dense bias", 2, 4352, 24, 64, bf, "dense_shared"))
    if only == "attn_c5_vector":
        out.append(attention_case(torch, "attn_c5_vector: (2,4352,24,64) bf16, the key mask as a (B,1,1,T) vector", 2, 4352, 24, 64, bf, "vector"))
    if only == "attn_c5_maskfull":
        out.append(attention_case(torch, "attn_c5_maskfull: (2,4352,24,64) bf16, the key mask written out as (B,H,T,T)", 2, 4352, 24, 64, bf,
                                  "mask_full"))
    # kernel quality at head dim 128 without the help of -inf blocks: a finite bias of config 4's shape, and a causal launch
    if want("attn_c4_finite"):
        out.append(attention_case(torch, "attn_c4_finite: (2,2048,16,128) fp16 (B,H,T,T) finite bias (no -inf blocks)", 2, 2048, 16, 128,
                                  torch.float16, "dense_full"))
    if want("attn_causal128"):
        out.append(attention_case(torch, "attn_causal128: (2,8192,16,128) fp16 causal, no bias (FLOPs of the lower triangle)", 2, 8192, 16,
                                  128, torch.float16, None, iters=10, causal=True))
    # buffer sets are sized so that their sum exceeds the 256 MB Infinity Cache
    if want("rms_c1"):
        out.append(rms_case(torch, "rms_c1: FusedRMSNorm (4,1024,1024) fp32 fwd+bwd", 4, [(1024, 1024)], torch.float32, 12, with_cpu=with_cpu))
    if want("rms2_c5"):
        out.append(rms_case(torch, "rms2_c5: FusedRMSNorm2 (2,4096,1536)+(2,256,1536) bf16 fwd+bwd", 2,
                            [(4096, 1536), (256, 1536)], bf, 12, with_cpu=with_cpu))
    if want("rms_wide"):
        out.append(rms_case(torch, "rms_wide: FusedRMSNorm (8,4096,4096) bf16 fwd+bwd", 8, [(4096, 4096)], bf, 3, with_api=False))
    if want("rope_c2"):
        out.append(rope_case(torch, "rope_c2: RoPE q,k (8,2048,16,64) bf16, R=32, forward + backward rotation", 8, 2048, 16, 64, 32, bf, 4))
    if want("l2x2_c5"):
        out.append(l2_case(torch, "l2x2_c5: FusedL2Normalize2 (2,4096,1536)+(2,256,1536) bf16 fwd+bwd", 2, [(4096, 1536), (256, 1536)], bf, 12))
    if want("headln_c5"):
        out.append(head_ln_case(torch, "headln_c5: FusedHeadLayerNorm q,k (2,4352,24,64) bf16 fwd+bwd", 2, 4352, 24, 64, bf, 6, with_cpu=with_cpu))
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU; --gpus {args.gpus} is not supported (use --gpus 1).", file=sys.stderr)
        sys.exit(2)
    import torch

    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.only:
        print(json.dumps({"extra": extras(torch, args.only, with_cpu=not args.skip_cpu)}))
        return
    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    B, T, H, D = 8, 2048, 16, 64
    pe, sets = make_ln_rope_sets(torch, 4, B, T, H, D)
    fns = ln_rope_steps(torch, pe, sets)
    wall_ms, gpu_ms, fwd, bwd, event_gap = timed_loop(torch, fns, args.steps, args.warmup)
    step_bytes = 5 * 2 * B * T * H * D * 2          # fwd: read x, write y; bwd: read x, dy, write dx (q and k)
    bwd_bytes = 3 * 2 * B * T * H * D * 2
    fwd_bytes = 2 * 2 * B * T * H * D * 2
    # the K steps are bracketed by synchronisations AND by two events on the launch stream; `value` is priced on the
    # event span (what the GPU needed for exactly K steps).  The wall-clock figure of the same K steps, which adds the
    # host's wake-up after the last step (tens of microseconds once, i.e. a few per cent of 20 steps of 60 us, nothing
    # at 1000 steps), is reported beside it in `timing`.
    ms = gpu_ms
    bwd_avg, fwd_avg = statistics.mean(bwd), statistics.mean(fwd)
    achieved = bwd_bytes / bwd_avg / 1e6
    prof = profile_figures()
    traffic = int(prof["traffic_bytes_per_launch"]) if "traffic_bytes_per_launch" in prof else None
    rocprof_us = float(prof["rocprof_avg_launch_us"]) if "rocprof_avg_launch_us" in prof else None
    result = {
        "metric": "attn fwd+bwd TFLOP/s (% MFMA peak); norm/RoPE GB/s (% HBM peak)",
        "value": round(step_bytes / ms / 1e6, 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 in/out, f32 arithmetic",
        "data": "synthetic",
        "config": {"workload": "configs[1]: FusedLNRoPE fwd+bwd, q,k (8,2048,16,64) bf16, heads_second=False, eps=1e-5, "
                               "R=32, theta=10000, cutoff (2048,2048), P=2049",
                   "step": "rgd_ln_rope_qk_fwd + rgd_ln_rope_qk_bwd through the C ABI, 4 rotating buffer sets (1.07 GB)",
                   "algorithmic_bytes_per_step": step_bytes},
        # achieved / frac: algorithmic bytes of a launch over the kernel's average duration in the committed rocprofv3
        # kernel trace of this same command (reproducible: profiles/...), or over the live event figure when the summary is
        # missing.  live_hip_events: the same launch timed in this run with an event before and after it; an event pair
        # with nothing between costs `event_gap_ms`, and an interval holds between none and all of it, so the kernel's
        # duration lies between the two figures given.
        "roofline": {"bound": "hbm", "kernel": "head_rows_kernel<bf16, LNROPE_BWD> (rgd_ln_rope_qk_bwd)",
                     "achieved": round(bwd_bytes / rocprof_us / 1e3 if rocprof_us else achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s",
                     "frac": round((bwd_bytes / rocprof_us / 1e3 if rocprof_us else achieved) / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "algorithmic_bytes_per_launch": bwd_bytes,
                     "avg_launch_ms": round(rocprof_us / 1e3 if rocprof_us else bwd_avg, 5),
                     "duration_source": ("rocprofv3 --kernel-trace --stats of this command, " + PROFILE_SUMMARY +
                                         " (measured at " + str(prof.get("measured_at")) + ")") if rocprof_us else
                                        "HIP events of this run (no profile summary found)",
                     "live_hip_events": {"interval_ms": round(bwd_avg + event_gap, 5), "event_gap_ms": round(event_gap, 5),
                                         "frac_if_no_gap_inside": round(bwd_bytes / (bwd_avg + event_gap) / 1e6 / HBM_PEAK_GBS, 4),
                                         "frac_if_whole_gap_inside": round(achieved / HBM_PEAK_GBS, 4),
                                         "fwd_interval_ms": round(fwd_avg + event_gap, 5)},
                     "fwd_kernel": {"rocprof_avg_launch_us": float(prof["rocprof_fwd_avg_launch_us"]) if "rocprof_fwd_avg_launch_us" in prof else None,
                                    "frac": round(fwd_bytes / float(prof["rocprof_fwd_avg_launch_us"]) / 1e3 / HBM_PEAK_GBS, 4)
                                    if "rocprof_fwd_avg_launch_us" in prof else None}},
        "timing": {"wall_ms_per_step": round(wall_ms, 5), "gpu_event_span_ms_per_step": round(gpu_ms, 5),
                   "value_from": "gpu_event_span_ms_per_step", "value_on_wall_clock": round(step_bytes / wall_ms / 1e6, 1)},
    }
    if not args.skip_cpu:
        result["cpu_baseline"] = cpu_baseline_ln_rope(torch)
    else:
        result["cpu_baseline"] = None
    if not args.skip_extra:
        del sets, fns
        torch.cuda.empty_cache()
        if not args.skip_cpu:
            result["torch_eager_gpu"] = torch_eager_ln_rope(torch)
            torch.cuda.empty_cache()
        result["extra"] = extras(torch, with_cpu=not args.skip_cpu)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
