"""CPU oracle for the rgd-triton operator set.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file; it is used by
tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker the HIP
kernels are compared against.  It restates, in plain PyTorch eager on the CPU, the algorithms
of the reference operators.  Every function cites the reference lines it follows
(paths relative to the reference checkout).

Forward functions follow the PyTorch reference math the reference's own tests compare against;
the closed-form backward functions follow the reference's kernels.  How each one is pinned
(tests/test_oracle_pinning.py):

  rms_fwd / rms_bwd            torch.nn.functional.rms_norm + autograd (fp64), hand loop on tiny input
  l2_fwd / l2_bwd              torch.nn.functional.normalize + autograd (fp64) for rows with |x| >= eps;
                               clamped rows: closed form y = x/eps
  head_ln_fwd / head_ln_bwd    torch.nn.functional.layer_norm + autograd (fp64)
  rope_fwd / rope_bwd          complex-number rotation identity, norm preservation, exact copy for
                               cutoff 0 / channels >= R, autograd transpose for pair-duplicated tables
  ln_rope_fwd / ln_rope_bwd    composition of the two pinned halves + autograd (fp64)
  attention_fwd / attention_bwd  brute-force python loops in fp64 on tiny inputs, torch.softmax /
                               torch.logsumexp, autograd (fp64, including the bias gradient in every broadcast
                               form), bias-broadcast equivalence
  attention_lowp               in fp64 it equals attention_fwd and the brute-force loops for every bias form,
                               causal or not, and its autograd gradients equal attention_bwd; in bf16 / fp16 its
                               error lies in a measured band around the rounding error of the exact result
  rotary_table                 sin^2 + cos^2 = 1, pair duplication, angle(t) = t * theta^(-2i/R)

No function here is "parity unpinned".
"""
import math

import torch

# ----------------------------------------------------------------------------------------------
# tolerances: (rtol, atol) per dtype, in that order, exactly as the reference's tests define them
# ----------------------------------------------------------------------------------------------


def get_tolerance(dtype, op="default"):
    """(rtol, atol) used by the reference's tests.

    default: tests/test_rms.py:15-26, tests/test_head_layernorm.py:15-26,
             tests/test_l2normalize.py:15-26 (bf16 atol is 2e-5 in test_rms.py, 1e-5 elsewhere)
    rope:    tests/test_head_rope.py:211-223
    ln_rope: tests/test_fused_ln_rope.py:220-233
    """
    if op == "rope":
        table = {torch.float32: (1.3e-6, 1e-5), torch.float16: (1e-3, 1e-3), torch.bfloat16: (1.6e-2, 1e-5)}
    elif op == "ln_rope":
        table = {torch.float32: (1.3e-6, 1e-5), torch.float16: (1e-3, 1e-2), torch.bfloat16: (1.6e-2, 1e-3)}
    elif op == "rms":
        table = {torch.float32: (1.3e-6, 1e-5), torch.float16: (1e-3, 1e-5), torch.bfloat16: (1.6e-2, 2e-5)}
    else:
        table = {torch.float32: (1.3e-6, 1e-5), torch.float16: (1e-3, 1e-5), torch.bfloat16: (1.6e-2, 1e-5)}
    if dtype not in table:
        raise ValueError(f"Unhandled dtype: {dtype}")
    return table[dtype]


# ----------------------------------------------------------------------------------------------
# RMSNorm
# ----------------------------------------------------------------------------------------------


def _expand_w(w, x):
    """Weight broadcast rule of RMS_Func.forward (normalization/rmsnorm_cached.py:582-589):
    (C,) or (1,1,C) is shared by every batch element, (B,1,C) is per batch element."""
    if w.ndim == 1:
        return w.view(1, 1, -1).expand(x.shape[0], 1, -1), True
    if w.shape[0] == 1:
        return w.expand(x.shape[0], -1, -1), True
    return w, False


def rms_fwd(x, w, eps=1e-6, compute_dtype=torch.float32):
    """y = x * rsqrt(mean(x^2) + eps) * w, computed in fp32 and cast to x.dtype.

    Follows tests/test_rms.py:29-38 (F.rms_norm(x.float(), (C,), None, eps) * w.float()) and the
    kernel normalization/rmsnorm_cached.py:59-101."""
    xf = x.to(compute_dtype)
    we, _ = _expand_w(w.to(compute_dtype), x)
    rrms = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xf * rrms * we).to(x.dtype)


def rms_bwd(dy, x, w, eps=1e-6, compute_dtype=torch.float32):
    """Closed-form backward of rms_fwd, following normalization/rmsnorm_cached.py:195-236:
        xhat = x * rrms
        dx   = (dy * w - xhat * mean(xhat * dy * w)) * rrms
        dw   = sum over rows of xhat * dy      (per batch element; summed over batch when shared,
                                                rmsnorm_cached.py:623-625)
    dw is accumulated in compute_dtype and cast once to w.dtype."""
    xf, dyf = x.to(compute_dtype), dy.to(compute_dtype)
    we, shared = _expand_w(w.to(compute_dtype), x)
    rrms = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    xhat = xf * rrms
    inner = (xhat * dyf * we).mean(dim=-1, keepdim=True)
    dx = (dyf * we - xhat * inner) * rrms
    dw = (xhat * dyf).sum(dim=1, keepdim=True)  # (B,1,C)
    if shared:
        dw = dw.sum(dim=0)  # (1,C)
    return dx.to(x.dtype), dw.reshape(w.shape).to(w.dtype)


# ----------------------------------------------------------------------------------------------
# L2 normalize
# ----------------------------------------------------------------------------------------------


def l2_fwd(x, eps=1e-6, compute_dtype=torch.float32):
    """y = x / max(||x||_2, eps) along the last dim (tests/test_l2normalize.py:28-34,
    F.normalize(x.float(), p=2, eps=eps, dim=-1)); the kernel writes it as
    rlen = 1/eps if len < eps else 1/len (normalization/l2normalize_cached.py:72-77)."""
    xf = x.to(compute_dtype)
    ln = xf.pow(2).sum(dim=-1, keepdim=True).sqrt()
    rlen = torch.where(ln < eps, torch.full_like(ln, 1.0 / eps), 1.0 / ln)
    return (xf * rlen).to(x.dtype)


def l2_bwd(dy, x, eps=1e-6, compute_dtype=torch.float32):
    """dx = (dy - xhat * sum(xhat * dy)) * rlen with xhat = x * rlen
    (normalization/l2normalize_cached.py:203-231).  The same expression is used for clamped rows
    (len < eps); the exact clamped gradient dy/eps is commented out in the reference (:231)."""
    xf, dyf = x.to(compute_dtype), dy.to(compute_dtype)
    ln = xf.pow(2).sum(dim=-1, keepdim=True).sqrt()
    rlen = torch.where(ln < eps, torch.full_like(ln, 1.0 / eps), 1.0 / ln)
    xhat = xf * rlen
    inner = (xhat * dyf).sum(dim=-1, keepdim=True)
    return ((dyf - xhat * inner) * rlen).to(x.dtype)


# ----------------------------------------------------------------------------------------------
# per-head LayerNorm (no affine)
# ----------------------------------------------------------------------------------------------


def head_ln_fwd(x, eps=1e-6, compute_dtype=torch.float32):
    """y = (x - mean) * rsqrt(var + eps) over the last (head) dim, biased variance, no affine
    (tests/test_head_layernorm.py:28-43; kernel normalization/head_layernorm_cached.py:60-85).
    The layout (heads_second or not) does not matter: rows are the last dim."""
    xf = x.to(compute_dtype)
    mu = xf.mean(dim=-1, keepdim=True)
    xc = xf - mu
    rstd = torch.rsqrt(xc.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xc * rstd).to(x.dtype)


def head_ln_bwd(dy, x, eps=1e-6, compute_dtype=torch.float32, out_dtype=None):
    """dx = (dy - xhat * mean(xhat * dy) - mean(dy)) * rstd
    (normalization/head_layernorm_cached.py:170-199; rope/fused_ln_rope_cached.py:88-114)."""
    xf, dyf = x.to(compute_dtype), dy.to(compute_dtype)
    mu = xf.mean(dim=-1, keepdim=True)
    xc = xf - mu
    rstd = torch.rsqrt(xc.pow(2).mean(dim=-1, keepdim=True) + eps)
    xhat = xc * rstd
    inner = (xhat * dyf).mean(dim=-1, keepdim=True)
    mdy = dyf.mean(dim=-1, keepdim=True)
    return ((dyf - xhat * inner - mdy) * rstd).to(out_dtype or x.dtype)


# ----------------------------------------------------------------------------------------------
# RoPE
# ----------------------------------------------------------------------------------------------


def rotary_table(num_pos, rot_dim, theta=10000.0, dtype=torch.float32):
    """pos_emb (2, num_pos, rot_dim): [0] = sin, [1] = cos, angle[t, i] = t * theta^(-2i/rot_dim),
    each value duplicated over the channel pair (2i, 2i+1) -- the 1-D analogue of the pair-duplicated
    table the reference's tests build (tests/test_head_rope.py:136,146,177: inv_freq, stack(sin, cos),
    repeat 'n d -> n (d j)', j=2)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot_dim, 2, dtype=torch.float32) / rot_dim))
    ang = torch.arange(num_pos, dtype=torch.float32)[:, None] * inv_freq[None, :]
    sin = ang.sin().repeat_interleave(2, dim=-1)
    cos = ang.cos().repeat_interleave(2, dim=-1)
    return torch.stack([sin, cos]).to(dtype)


def axial_rotary_table(emb_len, rot_dim, max_freq=32.0, dtype=torch.float32):
    """The 2-D axial table of tests/test_head_rope.py:128-190 (AxialRotaryEmbedding(RDIM//2,
    max_freq) on an emb_len x emb_len grid), flattened to (2, emb_len^2, rot_dim): the first
    rot_dim/2 channels rotate with the x coordinate, the rest with the y coordinate."""
    ch = rot_dim // 2
    inv_freq = 1.0 / (max_freq ** (torch.arange(0, ch, 2, dtype=torch.float32) / ch))
    pos = torch.arange(emb_len, dtype=torch.float32)
    ang = pos[:, None] * inv_freq[None, :]  # (L, ch/2)
    ax = ang[None, :, :].expand(emb_len, emb_len, -1)  # x varies along dim 1
    ay = ang[:, None, :].expand(emb_len, emb_len, -1)  # y varies along dim 0
    a = torch.cat([ax, ay], dim=-1).reshape(emb_len * emb_len, -1)  # (L*L, ch)
    sin = a.sin().repeat_interleave(2, dim=-1)
    cos = a.cos().repeat_interleave(2, dim=-1)
    return torch.stack([sin, cos]).to(dtype)


def _rot_fwd(x):
    # rotate_every_two of tests/test_head_rope.py:10-15: (x0, x1) -> (-x1, x0)
    x1, x2 = x[..., ::2], x[..., 1::2]
    return torch.stack((-x2, x1), dim=-1).flatten(-2)


def _rot_bwd(x):
    # the kernel's IS_BWD rotation, rope/head_rope_cached.py:35-40: (x0, x1) -> (x1, -x0)
    x1, x2 = x[..., ::2], x[..., 1::2]
    return torch.stack((x2, -x1), dim=-1).flatten(-2)


def _resolve_cutoff(seq_cutoff, tq, tk):
    # rope/head_rope_cached.py:193-201
    if seq_cutoff is None:
        return tq, tk
    if isinstance(seq_cutoff, (tuple, list)):
        return seq_cutoff[0], seq_cutoff[1]
    return seq_cutoff, seq_cutoff


def _rope_one(x, pos_emb, cutoff, heads_second, backward, compute_dtype):
    """x: (B,h,T,d) if heads_second else (B,T,h,d).  Rotates channels < R of tokens < cutoff with
    out = x*cos + rot(x)*sin, where sin/cos are taken at the OUTPUT channel
    (rope/head_rope_cached.py:45-51); identity elsewhere."""
    xf = x.to(compute_dtype)
    tdim = 2 if heads_second else 1
    T = x.shape[tdim]
    R = pos_emb.shape[-1]
    n = max(0, min(int(cutoff), T))
    sin = pos_emb[0, :T].to(compute_dtype)
    cos = pos_emb[1, :T].to(compute_dtype)
    if heads_second:
        sin, cos = sin[None, None], cos[None, None]  # (1,1,T,R)
    else:
        sin, cos = sin[None, :, None], cos[None, :, None]  # (1,T,1,R)
    xr = xf[..., :R]
    rot = _rot_bwd(xr) if backward else _rot_fwd(xr)
    out_r = xr * cos + rot * sin
    tok = torch.arange(T).view([1, 1, T, 1] if heads_second else [1, T, 1, 1])
    out_r = torch.where(tok < n, out_r, xr)
    return torch.cat([out_r, xf[..., R:]], dim=-1)


def rope_fwd(q, k, pos_emb, seq_cutoff=None, heads_second=True, compute_dtype=torch.float32):
    """RoPE on the first R channels and first cutoff tokens of q and k
    (tests/test_head_rope.py:21-124 with rotate_every_two :10-18; kernel rope/head_rope_cached.py:7-52).
    Computed in compute_dtype and rounded once to the input dtype."""
    tdim = 2 if heads_second else 1
    cq, ck = _resolve_cutoff(seq_cutoff, q.shape[tdim], k.shape[tdim])
    qo = _rope_one(q, pos_emb, cq, heads_second, False, compute_dtype).to(q.dtype)
    ko = _rope_one(k, pos_emb, ck, heads_second, False, compute_dtype).to(k.dtype)
    return qo, ko


def rope_bwd(dqo, dko, pos_emb, seq_cutoff=None, heads_second=True, compute_dtype=torch.float32):
    """Backward as the reference kernel computes it: the same transform with the rotation sign
    flipped (rope/head_rope_cached.py:35-40, called with is_bwd=True at :305-317).  This equals the
    exact transpose whenever sin/cos are equal within each channel pair."""
    tdim = 2 if heads_second else 1
    cq, ck = _resolve_cutoff(seq_cutoff, dqo.shape[tdim], dko.shape[tdim])
    dq = _rope_one(dqo, pos_emb, cq, heads_second, True, compute_dtype).to(dqo.dtype)
    dk = _rope_one(dko, pos_emb, ck, heads_second, True, compute_dtype).to(dko.dtype)
    return dq, dk


def ln_rope_fwd(q, k, pos_emb, seq_cutoff=None, heads_second=True, eps=1e-6, compute_dtype=torch.float32):
    """Head LayerNorm then RoPE, all in fp32 registers, one rounding at the end
    (tests/test_fused_ln_rope.py:73-124 with upcast=True; kernel rope/fused_ln_rope_cached.py:198-240)."""
    tdim = 2 if heads_second else 1
    cq, ck = _resolve_cutoff(seq_cutoff, q.shape[tdim], k.shape[tdim])
    qn = head_ln_fwd(q.to(compute_dtype), eps, compute_dtype)
    kn = head_ln_fwd(k.to(compute_dtype), eps, compute_dtype)
    qo = _rope_one(qn, pos_emb, cq, heads_second, False, compute_dtype).to(q.dtype)
    ko = _rope_one(kn, pos_emb, ck, heads_second, False, compute_dtype).to(k.dtype)
    return qo, ko


def ln_rope_bwd(dqo, dko, q, k, pos_emb, seq_cutoff=None, heads_second=True, eps=1e-6,
                compute_dtype=torch.float32):
    """Inverse-rotate dy, then LayerNorm backward (rope/fused_ln_rope_cached.py:353-375)."""
    tdim = 2 if heads_second else 1
    cq, ck = _resolve_cutoff(seq_cutoff, q.shape[tdim], k.shape[tdim])
    gq = _rope_one(dqo, pos_emb, cq, heads_second, True, compute_dtype)
    gk = _rope_one(dko, pos_emb, ck, heads_second, True, compute_dtype)
    dq = head_ln_bwd(gq, q, eps, compute_dtype, out_dtype=dqo.dtype)
    dk = head_ln_bwd(gk, k, eps, compute_dtype, out_dtype=dko.dtype)
    return dq, dk


# ----------------------------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------------------------


def _scores(q, k, bias, causal, softmax_scale, compute_dtype):
    B, Tq, h, d = q.shape
    Tk = k.shape[1]
    scale = softmax_scale or 1.0 / math.sqrt(d)  # flash_attn_triton_cached.py:768 (0.0 -> default)
    s = torch.einsum("bthd,bshd->bhts", q.to(compute_dtype), k.to(compute_dtype)) * scale
    if bias is not None:
        s = s + bias.to(compute_dtype)  # broadcast over leading dims and (1,Tk) rows, :779-788
    if causal:
        # top-left aligned: key index <= query index is kept (flash_attn_triton_cached.py:149-150)
        keep = torch.arange(Tq)[:, None] >= torch.arange(Tk)[None, :]
        s = s.masked_fill(~keep, float("-inf"))
    return s, scale


def attention_fwd(q, k, v, bias=None, causal=False, softmax_scale=None, compute_dtype=torch.float32):
    """O = softmax(scale * Q K^T + bias) V and LSE = logsumexp of the scores.

    q (B,Tq,h,d), k/v (B,Tk,h,d), bias broadcastable to (B,h,Tq,Tk).  Follows attention_ref,
    tests/test_flash_attn.py:18-62 (upcast=True), and for LSE the kernel's running logsumexp,
    flash_attn_triton_cached.py:174-214.  Returns (o in q.dtype, lse fp32 (B,h,Tq)).
    A row whose scores are all -inf yields o = 0 and lse = -inf (the reference kernel would give
    NaN there; its tests never produce such a row)."""
    s, _ = _scores(q, k, bias, causal, softmax_scale, compute_dtype)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)[..., None])
    p = torch.where(torch.isinf(lse)[..., None], torch.zeros_like(p), p)
    o = torch.einsum("bhts,bshd->bthd", p, v.to(compute_dtype))
    return o.to(q.dtype), lse.to(torch.float32)


def attention_bwd(do, q, k, v, bias=None, causal=False, softmax_scale=None, compute_dtype=torch.float32,
                  with_dbias=False):
    """Closed-form gradients as the reference kernels compute them
    (flash_attn_triton_cached.py:249-292 and :426-571):
        delta = rowsum(O * dO);  P = exp(S - LSE);  dV = P^T dO;  dP = dO V^T;
        dS = P * (dP - delta) * scale;  dK = dS^T Q;  dQ = dS K
    Everything in compute_dtype (no intermediate rounding).  with_dbias adds the gradient of the bias, which the
    reference does not provide (:1107): dS / scale, summed over the dimensions the bias broadcasts."""
    s, scale = _scores(q, k, bias, causal, softmax_scale, compute_dtype)
    lse = torch.logsumexp(s, dim=-1)
    dead = torch.isinf(lse)
    p = torch.exp(s - torch.where(dead, torch.zeros_like(lse), lse)[..., None])
    p = torch.where(dead[..., None], torch.zeros_like(p), p)
    vf, dof = v.to(compute_dtype), do.to(compute_dtype)
    o = torch.einsum("bhts,bshd->bthd", p, vf)
    delta = (o * dof).sum(dim=-1).permute(0, 2, 1)  # (B,h,Tq)
    dv = torch.einsum("bhts,bthd->bshd", p, dof)
    dp = torch.einsum("bthd,bshd->bhts", dof, vf)
    ds = p * (dp - delta[..., None]) * scale
    dk = torch.einsum("bhts,bthd->bshd", ds, q.to(compute_dtype))
    dq = torch.einsum("bhts,bshd->bthd", ds, k.to(compute_dtype))
    if not with_dbias:
        return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)
    db = p * (dp - delta[..., None])
    dims = [i for i in range(4) if bias.shape[i] == 1 and db.shape[i] != 1]
    if dims:
        db = db.sum(dim=dims, keepdim=True)
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), db.to(bias.dtype)


def attention_lowp(q, k, v, bias=None, causal=False):
    """The low-precision PyTorch run the reference's tests use as their error bar
    (attention_ref with upcast=False, reorder_ops=True; tests/test_flash_attn.py:51-62): all math
    in the input dtype, k scaled instead of q, probabilities rounded to v.dtype."""
    d = q.shape[-1]
    s = torch.einsum("bthd,bshd->bhts", q, k / math.sqrt(d))
    if bias is not None:
        s = s + bias
    if causal:
        keep = torch.arange(q.shape[1])[:, None] >= torch.arange(k.shape[1])[None, :]
        s = s.masked_fill(~keep, float("-inf"))
    p = torch.softmax(s, dim=-1).to(v.dtype)
    return torch.einsum("bhts,bshd->bthd", p, v).to(q.dtype)
