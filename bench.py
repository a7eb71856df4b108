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
`cpu_baseline` = the CPU oracle timed on this host on a bounded sample, and `extra` with the other
BASELINE configurations (attention TFLOP/s, RMSNorm2 / head LayerNorm GB/s) and the Module-API timing.
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

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this file (profiles/), scaled by a copy kernel of known size; None until measured for a workload.
MEASURED_TRAFFIC = {}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
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
    [fwd, bwd] given an event recorder.  Returns (wall ms per step, fwd ms list, bwd ms list)."""
    n = len(step_fns)
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
    # separate pass and not the one `value` comes from)
    evs = []
    for i in range(steps):
        rec = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        step_fns[(i + steps) % n](rec)
        evs.append(rec)
    torch.cuda.synchronize()
    fwd = [e[0].elapsed_time(e[1]) for e in evs]
    bwd = [e[1].elapsed_time(e[2]) for e in evs]
    return wall, gpu_span, fwd, bwd


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


def cpu_baseline_ln_rope(torch, B=2, T=2048, H=16, D=64, R=32, reps=3):
    """The CPU oracle (oracle/rgd_oracle.py, PyTorch eager fp32) on a batch-2 slice of the workload."""
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


# ------------------------------------------------------------------------------------------------
# extra workloads (reported under "extra", not the headline value)
# ------------------------------------------------------------------------------------------------
def time_api(torch, fn, iters=30, warmup=5):
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


def attention_case(torch, name, B, T, H, D, dtype, bias_kind, iters=20):
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
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    tqr = lib.rgd_attn_seqlen_q_rounded(T)
    lse = torch.empty(B, H, tqr, dtype=torch.float32, device="cuda")
    ws = torch.empty(lib.rgd_attn_bwd_workspace(B, H, T, T, D), dtype=torch.uint8, device="cuda")
    code = _hip.dtype_code(dtype)
    if bias is None:
        bdesc, bk, bd = _hip.Tensor4(None, 0, 0, 0), _hip.BIAS_NONE, _hip.RGD_F32
    else:
        be = bias.expand(B, H, T, T)
        bdesc, bk, bd = _hip.Tensor4(be.data_ptr(), be.stride(0), be.stride(1), be.stride(2)), _hip.BIAS_MATRIX, code
    t = {n: _hip.t4(x, False) for n, x in dict(q=q, k=k, v=v, do=do, o=o, dq=dq, dk=dk, dv=dv).items()}
    st = _hip.stream_ptr(q.device)
    scale = 1.0 / math.sqrt(D)

    def fwd():
        assert lib.rgd_attn_fwd(B, H, T, T, D, t["q"], t["k"], t["v"], bdesc, bk, bd, t["o"], lse.data_ptr(), code, 0,
                                scale, st) == 0, lib.rgd_last_error()

    def bwd():
        assert lib.rgd_attn_bwd(B, H, T, T, D, t["do"], t["q"], t["k"], t["v"], t["o"], lse.data_ptr(), bdesc, bk, bd,
                                t["dq"], t["dk"], t["dv"], code, 0, scale, ws.data_ptr(), ws.numel(), st) == 0, \
            lib.rgd_last_error()

    f_ms, b_ms = time_api(torch, fwd, iters, 3), time_api(torch, bwd, iters, 3)
    flops = 14.0 * B * H * T * T * D
    tot = f_ms + b_ms
    return {"workload": name, "fwd_ms": round(f_ms, 4), "bwd_ms": round(b_ms, 4),
            "tflops": round(flops / tot / 1e9, 2), "fwd_tflops": round(flops * 4 / 14 / f_ms / 1e9, 2),
            "bwd_tflops": round(flops * 10 / 14 / b_ms / 1e9, 2), "frac_mfma_peak": round(flops / tot / 1e9 / MFMA_PEAK_TFLOPS, 4)}


def rows_case(torch, name, make, nbytes, nsets=4, iters=40):
    """HBM-bound operator through the Module API + autograd, rotating buffer sets"""
    sets = [make(i) for i in range(nsets)]
    idx = [0]

    def run():
        s = sets[idx[0] % nsets]
        idx[0] += 1
        s()

    ms = time_api(torch, run, iters, 8)
    return {"workload": name, "ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1),
            "frac_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "path": "Module API + autograd (eager launches)"}


def extras(torch, only=""):
    import rgd_triton_amd as rgd

    out = []
    bf = torch.bfloat16

    def want(n):
        return not only or only == n

    if want("attn_c3"):
        out.append(attention_case(torch, "attn_c3: (4,4096,16,64) bf16 no bias", 4, 4096, 16, 64, bf, None))
    if want("attn_c4"):
        out.append(attention_case(torch, "attn_c4: (2,2048,16,128) fp16 full bias", 2, 2048, 16, 128, torch.float16, "full"))
    if want("attn_c5"):
        out.append(attention_case(torch, "attn_c5: (2,4352,24,64) bf16 broadcast bias", 2, 4352, 24, 64, bf, "broadcast"))

    if want("rms_c1"):
        def mk_rms(i):
            x = torch.randn(4, 1024, 1024, device="cuda", requires_grad=True)
            m = rgd.FusedRMSNorm(1024, device="cuda")
            dy = torch.randn_like(x)
            return lambda: torch.autograd.grad(m(x), (x, m.weight), dy)
        out.append(rows_case(torch, "rms_c1: FusedRMSNorm (4,1024,1024) fp32 fwd+bwd", mk_rms, 83886080, nsets=8))
    if want("rms2_c5"):
        def mk_rms2(i):
            x1 = torch.randn(2, 4096, 1536, device="cuda", dtype=bf, requires_grad=True)
            x2 = torch.randn(2, 256, 1536, device="cuda", dtype=bf, requires_grad=True)
            m = rgd.FusedRMSNorm2((1536, 1536), device="cuda", dtype=bf)
            d1, d2 = torch.randn_like(x1), torch.randn_like(x2)
            return lambda: torch.autograd.grad(m(x1, x2), (x1, x2, m.weight1, m.weight2), (d1, d2))
        out.append(rows_case(torch, "rms2_c5: FusedRMSNorm2 (2,4096,1536)+(2,256,1536) bf16 fwd+bwd", mk_rms2, 133693440, nsets=6))
    if want("headln_c5"):
        def mk_ln(i):
            q = torch.randn(2, 4352, 24, 64, device="cuda", dtype=bf, requires_grad=True)
            k = torch.randn(2, 4352, 24, 64, device="cuda", dtype=bf, requires_grad=True)
            m = rgd.FusedHeadLayerNorm()
            d1, d2 = torch.randn_like(q), torch.randn_like(k)
            return lambda: torch.autograd.grad(m(q, k, heads_second=False), (q, k), (d1, d2))
        out.append(rows_case(torch, "headln_c5: FusedHeadLayerNorm q,k (2,4352,24,64) bf16 fwd+bwd", mk_ln, 267386880, nsets=4))
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
        print(json.dumps({"extra": extras(torch, args.only)}))
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
    wall_ms, gpu_ms, fwd, bwd = timed_loop(torch, fns, args.steps, args.warmup)
    step_bytes = 5 * 2 * B * T * H * D * 2          # fwd: read x, write y; bwd: read x, dy, write dx (q and k)
    bwd_bytes = 3 * 2 * B * T * H * D * 2
    fwd_bytes = 2 * 2 * B * T * H * D * 2
    ms = max(wall_ms, gpu_ms)
    bwd_avg, fwd_avg = statistics.mean(bwd), statistics.mean(fwd)
    achieved = bwd_bytes / bwd_avg / 1e6
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
        "roofline": {"bound": "hbm", "kernel": "head_rows_kernel<bf16, LNROPE_BWD> (rgd_ln_rope_qk_bwd)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get("ln_rope_bwd_c2"),
                     "algorithmic_bytes_per_launch": bwd_bytes, "avg_launch_ms": round(bwd_avg, 5),
                     "fwd_kernel": {"achieved": round(fwd_bytes / fwd_avg / 1e6, 1), "avg_launch_ms": round(fwd_avg, 5),
                                    "frac": round(fwd_bytes / fwd_avg / 1e6 / HBM_PEAK_GBS, 4)}},
        "timing": {"wall_ms_per_step": round(wall_ms, 5), "gpu_event_span_ms_per_step": round(gpu_ms, 5)},
    }
    if not args.skip_cpu:
        result["cpu_baseline"] = cpu_baseline_ln_rope(torch)
    else:
        result["cpu_baseline"] = None
    if not args.skip_extra:
        del sets, fns
        torch.cuda.empty_cache()
        result["extra"] = extras(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
