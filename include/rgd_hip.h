/*
 * rgd_hip.h -- C ABI of librgd_hip.so: gfx950 (MI355X) HIP kernels for the rgd-triton operator set.
 *
 * Each entry point replaces one host launch wrapper of the reference (the function that sits
 * between a torch.autograd.Function and its @triton.jit kernels); the reference file:line is
 * given with every declaration (paths relative to the reference checkout, rgd_triton/triton/...).
 *
 * Conventions
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer owned by the caller.
 *     The library never allocates or frees device memory.
 *   - strides are in ELEMENTS (not bytes) and may be any value that keeps accesses in bounds;
 *     the last dimension of every tensor is unit stride.  A stride of 0 broadcasts.
 *   - dtype codes: RGD_F32 / RGD_F16 / RGD_BF16.  All statistics and accumulation are fp32.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls only enqueue
 *     work and return; they never synchronise.
 *   - return value 0 on success, negative rgd_status otherwise; rgd_last_error() returns a
 *     thread-local message for the last failure on the calling thread.
 *   - functions are re-entrant; the only state is the loaded code object and what rgd_init() caches.
 *   - stream capture: after rgd_init() has returned 0, every entry point makes no runtime call other than its
 *     kernel launches on `stream` (no allocation, copy, memset, attribute or device query, no
 *     hipGetLastError unless a launch has failed), so a sequence of calls may be recorded into a HIP graph.
 *     The one exception is rgd_rms_bwd_noalloc, which asks hipGetDevice for the current device on every call
 *     (its scratch array has one address per GPU); hipGetDevice is allowed under capture.  The workspace queries
 *     (rgd_*_workspace, rgd_attn_seqlen_q_rounded) and rgd_version / rgd_last_error touch no stream at all.
 *   - a launch that fails returns RGD_ERR_LAUNCH and is also cleared from the runtime's per-thread last error,
 *     so the caller's next hipGetLastError reports the caller's own work.
 */
#ifndef RGD_HIP_H
#define RGD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum rgd_dtype { RGD_F32 = 0, RGD_F16 = 1, RGD_BF16 = 2 };

enum rgd_status {
    RGD_OK = 0,
    RGD_ERR_INVALID = -1,     /* bad argument (shape, dtype code, null pointer)          */
    RGD_ERR_UNSUPPORTED = -2, /* valid but outside what the kernels cover                 */
    RGD_ERR_LAUNCH = -3,      /* hipLaunchKernel reported an error                        */
    RGD_ERR_WORKSPACE = -4    /* caller-provided workspace too small                      */
};

enum rgd_bias_kind { RGD_BIAS_NONE = 0, RGD_BIAS_VECTOR = 1, RGD_BIAS_MATRIX = 2 };

/* (B, T, C) tensor of rows; element (b, n, c) lives at ptr + b*stride_b + n*stride_n + c.
 * For a weight (B,1,C) only stride_b is used (0 = one weight shared by the batch). */
typedef struct rgd_tensor3 {
    void*   ptr;
    int64_t stride_b;
    int64_t stride_n;
} rgd_tensor3;

/* (B, H, T, D) tensor addressed by (batch, head, token) strides whatever its memory order:
 * heads_second=True passes (stride(0), stride(1), stride(2)), heads_second=False passes
 * (stride(0), stride(2), stride(1)) -- the reference resolves layouts the same way
 * (normalization/head_layernorm_cached.py:216-231). */
typedef struct rgd_tensor4 {
    void*   ptr;
    int64_t stride_b;
    int64_t stride_h;
    int64_t stride_n;
} rgd_tensor4;

/* library / ABI version (major*1000 + minor) and last error text.  No counterpart in the reference. */
int         rgd_version(void);
const char* rgd_last_error(void);

/* One-time set-up: caches the compute-unit count of the current device, sets the LDS size attribute of
 * every attention kernel and resolves the scratch array of rgd_rms_bwd_noalloc on that device.  Thread-safe and
 * idempotent; every entry point calls it on its own, so an explicit call is only needed before the first entry
 * point runs under stream capture (call it when the library is loaded).  Returns RGD_ERR_LAUNCH while the process
 * has no usable device (nothing is latched: a later call tries again), and the attention kernels' set-up status
 * otherwise; a failure there is reported again by every attention entry point and leaves the row kernels
 * (RMS, L2, head LayerNorm, RoPE) usable.  No counterpart in the reference (Triton configures kernels when it
 * compiles them). */
int rgd_init(void);

/* ------------------------------------------------------------------------------------------
 * RMSNorm  y = x * rsqrt(mean(x^2) + eps) * w        x (B,T,C), w (B,1,C) or shared
 * ------------------------------------------------------------------------------------------ */

/* replaces _rms_fwd, normalization/rmsnorm_cached.py:319-403 (kernel :6-103) */
int rgd_rms_fwd(int64_t B, int64_t T, int64_t C,
                const rgd_tensor3* x, const rgd_tensor3* w, const rgd_tensor3* y,
                int x_dtype, int w_dtype, float eps, void* stream);

/* Bytes of scratch the backward needs for the deterministic dw reduction (any contents on entry): one fp32
 * partial dw row per block, which a second small kernel adds in a fixed order.  Calls that may overlap
 * (different streams) need separate workspaces.  T2 = C2 = 0 for the one-tensor backward.  Stands where the
 * reference allocates its lock and bucket buffers, normalization/rmsnorm_cached.py:455-470. */
size_t rgd_rms_bwd_workspace(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2);

/* replaces _rms_bwd, normalization/rmsnorm_cached.py:406-569 (kernels :106-264 and :269-313):
 *   dx = (dy*w - xhat*mean(xhat*dy*w)) * rrms,   dw[b or shared] = sum_rows xhat*dy.
 * dw is (B,1,C) addressed with dw->stride_b when w_shared == 0, and a single (C) row holding the
 * sum over the batch when w_shared != 0 (the reference sums a (B,1,C) buffer on the host,
 * rmsnorm_cached.py:623-625).  dw is accumulated in fp32, in a fixed order, and stored in w_dtype.
 * Rows of any width (the reference loops over channel blocks, rmsnorm_cached.py:198-219). */
int rgd_rms_bwd(int64_t B, int64_t T, int64_t C,
                const rgd_tensor3* dy, const rgd_tensor3* x, const rgd_tensor3* w,
                const rgd_tensor3* dx, const rgd_tensor3* dw, int w_shared,
                int x_dtype, int w_dtype, float eps,
                void* workspace, size_t workspace_bytes, void* stream);

/* rgd_rms_bwd for callers that cannot allocate device memory and have no workspace to hand over (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, kernels and results (bit for bit) as rgd_rms_bwd, minus the workspace: the partial dw rows live
 * in a device array that is part of the library's code object (rgd_rms_bwd_noalloc_limit() bytes, 16 MiB, per GPU,
 * held until the process ends).  The call makes no hipMalloc / hipFree and uses no allocating routine.  Shapes
 * whose rgd_rms_bwd_workspace(B, T, C, 0, 0) exceeds the limit are refused with RGD_ERR_WORKSPACE.
 * All calls on one GPU share that array: calls that may overlap in time on one GPU (different streams or
 * threads) race on it; callers that need overlap use rgd_rms_bwd with a workspace each. */
size_t rgd_rms_bwd_noalloc_limit(void);
int rgd_rms_bwd_noalloc(int64_t B, int64_t T, int64_t C,
                        const rgd_tensor3* dy, const rgd_tensor3* x, const rgd_tensor3* w,
                        const rgd_tensor3* dx, const rgd_tensor3* dw, int w_shared,
                        int x_dtype, int w_dtype, float eps, void* stream);

/* replaces _fused_rms_fwd, normalization/fused_rmsnorm_cached.py:389-501 (kernel :6-125):
 * the two tensors are normalised in one launch as one virtual tensor; they share B and the dtype,
 * and have independent T, C and weights. */
int rgd_fused_rms_fwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2,
                      const rgd_tensor3* x1, const rgd_tensor3* w1, const rgd_tensor3* y1,
                      const rgd_tensor3* x2, const rgd_tensor3* w2, const rgd_tensor3* y2,
                      int x_dtype, int w1_dtype, int w2_dtype, float eps, void* stream);

/* replaces _fused_rms_bwd, normalization/fused_rmsnorm_cached.py:504-722 (kernels :128-319, :324-383) */
int rgd_fused_rms_bwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2,
                      const rgd_tensor3* dy1, const rgd_tensor3* x1, const rgd_tensor3* w1,
                      const rgd_tensor3* dx1, const rgd_tensor3* dw1, int w1_shared,
                      const rgd_tensor3* dy2, const rgd_tensor3* x2, const rgd_tensor3* w2,
                      const rgd_tensor3* dx2, const rgd_tensor3* dw2, int w2_shared,
                      int x_dtype, int w1_dtype, int w2_dtype, float eps,
                      void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * L2 normalize  y = x / max(||x||, eps)              x (B,T,C)
 * ------------------------------------------------------------------------------------------ */

/* replaces _norm_fwd, normalization/l2normalize_cached.py:238-318 (kernel :5-124) */
int rgd_l2_fwd(int64_t B, int64_t T, int64_t C, const rgd_tensor3* x, const rgd_tensor3* y,
               int dtype, float eps, void* stream);

/* replaces _norm_bwd, normalization/l2normalize_cached.py:321-399 (kernel :130-234):
 *   dx = (dy - xhat*sum(xhat*dy)) * rlen, also for rows clamped by eps */
int rgd_l2_bwd(int64_t B, int64_t T, int64_t C, const rgd_tensor3* dy, const rgd_tensor3* x,
               const rgd_tensor3* dx, int dtype, float eps, void* stream);

/* replaces _fused_norm_fwd, normalization/fused_l2normalize_cached.py:251-351 (kernel :6-115) */
int rgd_fused_l2_fwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2,
                     const rgd_tensor3* x1, const rgd_tensor3* y1,
                     const rgd_tensor3* x2, const rgd_tensor3* y2,
                     int dtype, float eps, void* stream);

/* replaces _fused_norm_bwd, normalization/fused_l2normalize_cached.py:354-461 (kernel :121-247) */
int rgd_fused_l2_bwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2,
                     const rgd_tensor3* dy1, const rgd_tensor3* x1, const rgd_tensor3* dx1,
                     const rgd_tensor3* dy2, const rgd_tensor3* x2, const rgd_tensor3* dx2,
                     int dtype, float eps, void* stream);

/* ------------------------------------------------------------------------------------------
 * Per-head operators on query and key: q (B,H,Tq,D), k (B,H,Tk,D), one launch for both
 * ------------------------------------------------------------------------------------------ */

/* replaces _fused_ln_qk_fwd, normalization/head_layernorm_cached.py:204-309 (kernel :6-99):
 * LayerNorm over D without affine, D <= 256 */
int rgd_ln_qk_fwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                  const rgd_tensor4* q, const rgd_tensor4* k,
                  const rgd_tensor4* qo, const rgd_tensor4* ko,
                  int dtype, float eps, void* stream);

/* replaces _fused_ln_qk_bwd, normalization/head_layernorm_cached.py:311-413 (kernel :101-202):
 *   dx = (dy - xhat*mean(xhat*dy) - mean(dy)) * rstd; mean and rstd are recomputed from q, k */
int rgd_ln_qk_bwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                  const rgd_tensor4* q, const rgd_tensor4* k,
                  const rgd_tensor4* dqo, const rgd_tensor4* dko,
                  const rgd_tensor4* dq, const rgd_tensor4* dk,
                  int dtype, float eps, void* stream);

/* replaces combined_rope_fn, rope/head_rope_cached.py:160-274 (kernel :56-158, helper :7-52):
 *   out = x*cos + rot(x)*sin on channels < R of tokens < cutoff, copy elsewhere.
 * pos_emb is (2, P, R): [0] = sin, [1] = cos, strides pe_stride_s / pe_stride_n, dtype pe_dtype.
 * is_bwd flips the rotation sign (the reference's backward).  D <= 128, Tq < P and Tk < P.
 * Arithmetic is fp32 with one rounding to the tensor dtype.  In-place (qo == q) is allowed. */
int rgd_rope_qk(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                const rgd_tensor4* q, const rgd_tensor4* k,
                const rgd_tensor4* qo, const rgd_tensor4* ko,
                const void* pos_emb, int64_t P, int64_t R, int64_t pe_stride_s, int64_t pe_stride_n,
                int pe_dtype, int64_t q_cutoff, int64_t k_cutoff, int is_bwd,
                int dtype, void* stream);

/* replaces _fused_rope_ln_qk_fwd, rope/fused_ln_rope_cached.py:382-516 (kernel :117-240) */
int rgd_ln_rope_qk_fwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                       const rgd_tensor4* q, const rgd_tensor4* k,
                       const rgd_tensor4* qo, const rgd_tensor4* ko,
                       const void* pos_emb, int64_t P, int64_t R, int64_t pe_stride_s,
                       int64_t pe_stride_n, int pe_dtype, int64_t q_cutoff, int64_t k_cutoff,
                       int dtype, float eps, void* stream);

/* replaces _fused_rope_ln_qk_bwd, rope/fused_ln_rope_cached.py:518-647 (kernel :243-378):
 * inverse rotation of the upstream gradient, then the LayerNorm backward */
int rgd_ln_rope_qk_bwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                       const rgd_tensor4* q, const rgd_tensor4* k,
                       const rgd_tensor4* dqo, const rgd_tensor4* dko,
                       const rgd_tensor4* dq, const rgd_tensor4* dk,
                       const void* pos_emb, int64_t P, int64_t R, int64_t pe_stride_s,
                       int64_t pe_stride_n, int pe_dtype, int64_t q_cutoff, int64_t k_cutoff,
                       int dtype, float eps, void* stream);

/* ------------------------------------------------------------------------------------------
 * Attention with additive bias: q (B,Tq,H,D), k,v (B,Tk,H,D) given as (b,h,n) strides, D <= 128,
 * fp16 or bf16.  bias (B,H,Tq,Tk) by strides (stride_n = row stride; 0 rows for RGD_BIAS_VECTOR),
 * dtype = the tensor dtype or fp32, zero strides broadcast.
 * ------------------------------------------------------------------------------------------ */

/* rows of the LSE / delta buffers: Tq rounded up to a multiple of 64, as the reference allocates
 * them (flash_attn/flash_attn_triton_cached.py:790-792) */
int64_t rgd_attn_seqlen_q_rounded(int64_t Tq);

/* Tile classes of a bias, matrix or vector, that the heads share (stride_h == 0), head dims up to 64.  Such a bias is
 * usually a mask (0 / -inf), and the reference streams it tile by tile for every head and in every kernel
 * (flash_attn/flash_attn_triton_cached.py:151-175, :430-470).  One pass over the matrix leaves two bits per tile of 32
 * queries x 64 keys (all +0; all -inf; every row equal to the tile's first row; anything else); rgd_attn_fwd and
 * rgd_attn_bwd then run tiles that are all +0 like tiles without bias, leave all -inf tiles out and read the bias only
 * for the others (one row of it where the rows are equal).  An all-+0 bias gives the results of a call without bias
 * bit for bit.  In tiles that read the bias, the bias enters the logits before the q.k product is added instead of
 * after it, and the dQ kernel adds do.v^T to -delta instead of subtracting delta afterwards: against a call that uses no
 * classes, o, lse, dq, dk and dv agree to the last one or two bits of the tensor dtype, not bit for bit (a call is
 * still reproducible bit for bit against itself).  Batch elements in most of whose tiles the bias has to be read are run
 * by the ordinary kernels, bit for bit as without classes.  Both calls make the pass themselves, into the end of their
 * workspace, when bias_classes is NULL; a caller that runs several calls on one bias (a forward and its backward, or
 * every layer of a model that shares one mask) can make it once:
 *   rgd_attn_bias_classes_bytes  size of the classes for this bias and shape; 0 when they would not be used
 *                                (no bias, not shared by the heads, rows not 16-byte aligned, D > 64, H < 2, Tk < 64)
 *   rgd_attn_bias_classify       writes them (8-byte aligned buffer of that size), two kernel launches on `stream`
 * and pass the buffer as bias_classes.  The classes describe the bias VALUES: classify again when they change. */
size_t rgd_attn_bias_classes_bytes(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                                   const rgd_tensor4* bias, int bias_kind, int bias_dtype);
int rgd_attn_bias_classify(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                           const rgd_tensor4* bias, int bias_kind, int bias_dtype,
                           void* classes, size_t classes_bytes, void* stream);

/* replaces _flash_attn_forward, flash_attn/flash_attn_triton_cached.py:758-882 (kernel :21-246).
 * lse is fp32 (B, H, Tq_rounded); rows >= Tq are written as 0.  A query row whose logits are all
 * -inf gives o = 0 and lse = -inf.  bias_classes: NULL, or what rgd_attn_bias_classify wrote for this bias. */
int rgd_attn_fwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                 const rgd_tensor4* q, const rgd_tensor4* k, const rgd_tensor4* v,
                 const rgd_tensor4* bias, int bias_kind, int bias_dtype,
                 const rgd_tensor4* o, float* lse,
                 int dtype, int causal, float softmax_scale, const void* bias_classes,
                 void* workspace, size_t workspace_bytes, void* stream);

/* Optional scratch of rgd_attn_fwd (any contents on entry, 16-byte aligned).  With it, the query blocks of
 * the last, partly filled round of workgroups are split along the keys and merged by a second launch, which
 * fills the chip for grids that are not a multiple of the resident workgroups (and for small grids).  Its end holds the
 * tile classes of a head-shared bias when the caller passes none (8-byte aligned workspace).
 * workspace = NULL or a smaller buffer is legal: the call then splits less or not at all, and reads such a bias like
 * any other.  Results do not depend on scheduling; a split item sums its keys in a different grouping than an unsplit
 * one. */
size_t rgd_attn_fwd_workspace(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D);

/* Forms of the attention backward.
 *   RGD_ATTN_BWD_TWO_KERNEL  a dQ kernel (query blocks) and a dK/dV kernel (key blocks): seven matrix products for the
 *                            five of the mathematics, no atomics, every result reproducible bit for bit.
 *   RGD_ATTN_BWD_ONE_PASS    one key-block kernel that also produces dQ by fp32 atomic additions into a dq_accum in the
 *                            workspace (what the reference sketches with tl.atomic_add in its sequence-parallel
 *                            branch, flash_attn_triton_cached.py:553-565), head dims up to 64.  dK and dV are
 *                            reproducible bit for bit; dQ differs from run to run in its last bits (the reference's
 *                            own race test allows that, tests/test_flash_attn.py:368,383).
 *   RGD_ATTN_BWD_AUTO        the library's choice for the shape (the one-pass form only if the workspace holds
 *                            dq_accum). */
enum rgd_attn_bwd_mode { RGD_ATTN_BWD_AUTO = 0, RGD_ATTN_BWD_TWO_KERNEL = 1, RGD_ATTN_BWD_ONE_PASS = 2 };

/* bytes of scratch for rgd_attn_bwd in the given mode (any contents on entry, 16-byte aligned): delta, fp32
 * (B,H,Tq_rounded), which is required; for the one-pass form dq_accum, fp32 (B,H,Tq_rounded,D padded to 32 or 64),
 * required by RGD_ATTN_BWD_ONE_PASS; then room for the fp32 partial sums of split workgroups (as in
 * rgd_attn_fwd_workspace), which is optional: a smaller workspace is accepted and nothing is split; and, for head dims
 * above 64, two ints for every 32 query rows in which the dQ launch tells the dK/dV launch which keys those rows
 * see through a bias with -inf blocks (optional as well: without room for them the dK/dV launch looks at the bias
 * itself, with the same results); for head dims up to 64, the tile classes of a head-shared bias when the caller passes
 * none (optional as well). */
size_t rgd_attn_bwd_workspace(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, int mode);

/* replaces _flash_attn_backward, flash_attn/flash_attn_triton_cached.py:885-1075
 * (kernels :249-292 and :327-755): delta = rowsum(o*do), P recomputed from lse, dv = P^T do,
 * dS = P*(do v^T - delta)*scale, dk = dS^T q, dq = dS k.
 * dbias (NULL, or ptr NULL: none; the reference has none, flash_attn_triton_cached.py:1107) receives the bias
 * gradient P*(do v^T - delta) of every (query, key) pair in the bias dtype: a full (B,H,Tq,Tk) tensor by strides,
 * 16-byte aligned, rows at least Tk rounded up to 64 elements long, which the caller
 * sums over the dimensions its bias broadcasts.  Columns up to Tk rounded up to the kernel's key tile (64 for head
 * dims up to 64, 32 above) are written, the rest of a row is left as it was.  Every pair is rounded to the bias
 * dtype before the caller's sum sees it.  With causal != 0 the caller clears it first (key tiles past the
 * diagonal are not visited).  Two-kernel form only.  dq, dk, dv are written
 * in the tensor dtype from fp32 accumulators, each exactly once; in a fixed order except for dq in the one-pass
 * form (see rgd_attn_bwd_mode).  bias_classes: NULL, or what rgd_attn_bias_classify wrote for this bias (used by the
 * two-kernel form without a bias gradient). */
int rgd_attn_bwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                 const rgd_tensor4* dout, const rgd_tensor4* q, const rgd_tensor4* k,
                 const rgd_tensor4* v, const rgd_tensor4* o, const float* lse,
                 const rgd_tensor4* bias, int bias_kind, int bias_dtype,
                 const rgd_tensor4* dq, const rgd_tensor4* dk, const rgd_tensor4* dv,
                 const rgd_tensor4* dbias,
                 int dtype, int causal, float softmax_scale, int mode, const void* bias_classes,
                 void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RGD_HIP_H */
