"""Shared pieces of the parity tests: seeded CPU input generation (the oracle and the GPU kernel see
the same bits) and the reference's comparison rules."""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

import rgd_oracle as oracle  # noqa: E402

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
DEV = "cuda"


def gen(seed):
    return torch.Generator().manual_seed(seed)


def gpu_gen(seed):
    """A generator on the GPU, for the repeat-and-compare tests: they have no oracle, and their batch-60 inputs take
    longer to draw on the host than their 250 repeats take on the GPU."""
    return torch.Generator(device=DEV).manual_seed(seed)


def randn(g, *shape, dtype=torch.float32, scale=1.0, shift=0.0):
    """N(shift, scale) drawn in fp32 where the generator lives (the CPU, unless it came from gpu_gen), then rounded
    to dtype."""
    return (torch.randn(*shape, generator=g, dtype=torch.float32, device=g.device) * scale + shift).to(dtype)


def dev(t):
    """t on the GPU with the same sizes, strides and storage offset.  `t.to("cuda")` makes a view with gaps
    contiguous, which would take the strided and unaligned layouts out of a test; here the whole underlying buffer
    is rebuilt on the GPU, NaN outside the view, so a read beyond the view shows up in the result."""
    if t.is_contiguous() or 0 in t.stride() or not t.is_floating_point():
        return t.to(DEV)
    n = t.untyped_storage().nbytes() // t.element_size()
    base = torch.full((n,), float("nan"), dtype=t.dtype, device=DEV)
    v = base.as_strided(t.size(), t.stride(), t.storage_offset())
    v.copy_(t)
    return v


def to_gpu(*ts, requires_grad=False):
    out = [dev(t).detach().requires_grad_(requires_grad) for t in ts]
    return out if len(out) > 1 else out[0]


def assert_close(actual, expected, dtype, op="default", name="", atol_scale=1.0):
    rtol, atol = oracle.get_tolerance(dtype, op)
    torch.testing.assert_close(actual.detach().cpu(), expected.detach().cpu(), rtol=rtol, atol=atol * atol_scale,
                               msg=lambda m: f"{name}: {m}")


def assert_close_allow_inf(actual, expected, dtype, name=""):
    """safe_assert_close_allow_inf of the reference's L2 tests (tests/test_l2normalize.py:54-111):
    NaN is forbidden, +-inf must sit at the same places, finite values compare within tolerance."""
    a, e = actual.detach().cpu().float(), expected.detach().cpu().float()
    assert not torch.isnan(a).any(), f"{name}: NaN in result"
    assert torch.equal(torch.isinf(a), torch.isinf(e)), f"{name}: inf pattern differs"
    fin = ~torch.isinf(e)
    rtol, atol = oracle.get_tolerance(dtype)
    torch.testing.assert_close(a[fin], e[fin], rtol=rtol, atol=atol, msg=lambda m: f"{name}: {m}")


RACE_ITERS = 250  # repeats of the reference's race-condition tests (tests/test_flash_attn.py:367, tests/test_rms.py:228)


def assert_repeats_bit_exact(fn, names, iters=RACE_ITERS):
    """Runs fn() (which returns GPU tensors) once, then `iters` more times, and requires every tensor of every repeat
    to have the bits of the first run.  Differing bits are collected on the GPU (xor of the integer views, so NaN
    equals NaN, or-ed into one accumulator per tensor: two launches per tensor and repeat, nothing allocated) and
    read back once at the end: the loop stays as dense as the reference's, which checks on the host every time."""
    ints = {1: torch.int8, 2: torch.int16, 4: torch.int32, 8: torch.int64}
    first = [t.detach().clone() for t in fn()]
    views = [t.view(ints[t.element_size()]) for t in first]
    acc = [torch.zeros_like(v) for v in views]
    tmp = [torch.empty_like(v) for v in views]
    for _ in range(iters):
        cur = fn()
        assert len(cur) == len(first)
        for a, b, x, t in zip(cur, views, acc, tmp):
            torch.bitwise_xor(a.detach().view(b.dtype), b, out=t)
            x.bitwise_or_(t)
    bad = [int((x != 0).sum().item()) for x in acc]  # elements that differed in some repeat
    assert not any(bad), {n: c for n, c in zip(names, bad) if c}
