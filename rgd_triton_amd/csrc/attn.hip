// Host side of the attention kernels: validation, dispatch and the extern "C" entry points.
#include "attn_fwd.h"
#include "attn_bwd.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

// kernel instantiations live in attn_f16.hip / attn_bf16.hip (attn_inst.h) so they compile in parallel
template <typename T> int dispatch_fwd(const AttnFwdParams& p, unsigned grid, hipStream_t s);
template <typename T> int dispatch_fwd_merge(const AttnFwdParams& p, unsigned items, hipStream_t s);
template <typename T> int dispatch_bwd_merge(const AttnBwdParams& p, unsigned items, int nt, hipStream_t s);
template <typename T, bool DQ> int dispatch_bwd(const AttnBwdParams& p, unsigned grid, hipStream_t s);
template <typename T> int dispatch_bwd_fused(const AttnBwdParams& p, unsigned grid, hipStream_t s);
template <typename T> int dispatch_bwd_fused_aux(const AttnBwdParams& p, int which, hipStream_t s);
// kernels that read the tile classes of a head-shared bias: attn_cls_f16.hip / attn_cls_bf16.hip; the pass that
// writes the classes: attn_classes.hip
template <typename T> int dispatch_fwd_cls(const AttnFwdParams& p, unsigned grid, hipStream_t s);
template <typename T, bool DQ> int dispatch_bwd_cls(const AttnBwdParams& p, unsigned grid, hipStream_t s);
int attn_classify(const void* bias, int64_t sb, int64_t sn, int bias_dtype, int nb, int64_t Tq, int64_t Tk, uint64_t* words,
                  hipStream_t s);

// 1: RGD_ATTN_BWD_AUTO takes the one-pass form where it exists
#ifndef RGD_ATTN_BWD_AUTO_ONE_PASS
#define RGD_ATTN_BWD_AUTO_ONE_PASS 0
#endif

namespace {

bool t4_vec_ok(const rgd_tensor4* t) {
    return rgd_aligned16(t->ptr) && (t->stride_b % 8) == 0 && (t->stride_h % 8) == 0 && (t->stride_n % 8) == 0;
}
AttnTensor at(const rgd_tensor4* t) {
    AttnTensor a;
    a.ptr = t ? t->ptr : nullptr;
    a.sb = t ? t->stride_b : 0;
    a.sh = t ? t->stride_h : 0;
    a.sn = t ? t->stride_n : 0;
    return a;
}

int attn_dpad(int64_t D) { return D <= 32 ? 32 : D <= 64 ? 64 : D <= 96 ? 96 : 128; }
// resident workgroups per compute unit of the forward kernel (its launch bounds and LDS use)
#ifndef RGD_GROUP_SHARED_BIAS
#define RGD_GROUP_SHARED_BIAS 1
#endif
int fwd_blocks_per_cu(int dpad, bool bias) { return (dpad <= 64 && !bias) ? 3 : 2; }
// bytes one part of a split forward item leaves behind: 128 rows of accumulators, exponent and row sum
size_t fwd_part_bytes(int dpad) { return (size_t)ATTN_BM * dpad * sizeof(float) + (size_t)ATTN_BM * 2 * sizeof(float); }

// resident workgroups per compute unit of the backward kernels, and the bytes a part of a split item leaves
int bwd_blocks_per_cu(int dpad) { return dpad <= 64 ? 2 : 1; }           // dK/dV kernel
int dq_blocks_per_cu(int dpad) { return (dpad <= 64 || dpad == 128) ? 2 : 1; }  // dQ kernel (32-key tiles at 128)
size_t bwd_part_bytes(int dpad, int tensors) { return (size_t)tensors * BWD_BM * dpad * sizeof(float); }
// key ranges the dQ launch leaves for the dK/dV launch (head dims above 64): two ints for every 32 query rows
int64_t bwd_rows32(int64_t Tq) { return (Tq + BWD_BM - 1) / BWD_BM * (BWD_BM / 32); }  // whole row blocks of the dQ launch
size_t bwd_ranges_bytes(int64_t B, int64_t H, int64_t Tq, int dpad) {
    return dpad > 64 ? (size_t)(B * H * bwd_rows32(Tq)) * 2 * sizeof(int) : 0;
}
size_t bwd_delta_bytes(int64_t B, int64_t H, int64_t Tq) { return (size_t)(B * H * rgd_attn_seqlen_q_rounded(Tq)) * sizeof(float); }
// one-pass form: fp32 dq_accum (B, H, Tq_rounded, DPAD) behind delta
size_t bwd_accum_bytes(int64_t B, int64_t H, int64_t Tq, int dpad) { return bwd_delta_bytes(B, H, Tq) * (size_t)dpad; }
// The form a call runs in.  AUTO takes the one-pass form where it exists (head dims up to 64) and the workspace has
// room for dq_accum; its dQ then depends on the arrival order of atomic additions (last-bit differences from run to
// run), dK and dV do not.  TWO_KERNEL is reproducible bit for bit.
bool bwd_one_pass(int mode, int64_t D, size_t workspace_bytes, size_t need) {
    if (mode == RGD_ATTN_BWD_TWO_KERNEL || D > 64) return false;
    if (mode == RGD_ATTN_BWD_ONE_PASS) return true;
    return RGD_ATTN_BWD_AUTO_ONE_PASS && workspace_bytes >= need;
}

// a vector bias is a matrix whose rows are all the same row
int64_t cls_row_stride(const rgd_tensor4* bias, int bias_kind) { return bias_kind == RGD_BIAS_VECTOR ? 0 : bias->stride_n; }
// Tile classes (attn_classes.h) pay for a bias (matrix or vector) that several heads share: one pass over it instead of
// one per head and kernel.  Head dims up to 64 (the kernels for wider heads have no registers for a second code path),
// rows the 16-byte loads can read, and a key count a wavefront can keep the classes of.
bool cls_eligible(int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* bias, int bias_kind, int bias_dtype) {
    if ((bias_kind != RGD_BIAS_MATRIX && bias_kind != RGD_BIAS_VECTOR) || !bias || bias->stride_h != 0 || H < 2 || D > 64 || Tq < 1 ||
        Tk < CLS_KEYS)
        return false;
    const int64_t per16 = bias_dtype == RGD_F32 ? 4 : 8;
    if (!rgd_aligned16(bias->ptr) || bias->stride_b % per16 != 0 || cls_row_stride(bias, bias_kind) % per16 != 0) return false;
    return cls_nwords(Tk) <= CLS_MAX_WORDS && cls_nrow32(Tq) <= CLS_MAX_ROWS;
}
int64_t cls_batches(int64_t B, const rgd_tensor4* bias) { return bias->stride_b == 0 ? 1 : B; }
BiasClasses cls_desc(const void* buffer, int64_t B, int64_t Tq, int64_t Tk, const rgd_tensor4* bias, int bias_kind) {
    return cls_layout(buffer, cls_batches(B, bias), Tq, Tk, cls_row_stride(bias, bias_kind) == 0);
}
// The classes a call works with: the caller's (bias_classes), or written here into the end of the workspace when it has
// room for them behind `fixed_bytes`; *room is what is left of the workspace in front of them.  Null: none.
const void* cls_for_call(const char* name, int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* bias,
                         int bias_kind, int bias_dtype, const void* bias_classes, void* workspace, size_t workspace_bytes,
                         size_t fixed_bytes, size_t* room, hipStream_t s, int* rc) {
    *rc = RGD_OK;
    if (!cls_eligible(H, Tq, Tk, D, bias, bias_kind, bias_dtype)) return nullptr;
    if (bias_classes) {
        if ((reinterpret_cast<uintptr_t>(bias_classes) & 7u) != 0) {
            rgd_set_error("%s: bias_classes must be 8-byte aligned", name);
            *rc = RGD_ERR_INVALID;
            return nullptr;
        }
        return bias_classes;
    }
    const size_t need = cls_bytes(cls_batches(B, bias), Tq, Tk);
    if (!workspace || workspace_bytes < fixed_bytes + need + 16) return nullptr;
    const size_t tail = (workspace_bytes - need) & ~(size_t)15;
    if (reinterpret_cast<uintptr_t>(workspace) & 7u) return nullptr;
    uint64_t* words = reinterpret_cast<uint64_t*>(static_cast<char*>(workspace) + tail);
    *rc = attn_classify(bias->ptr, bias->stride_b, cls_row_stride(bias, bias_kind), bias_dtype, (int)cls_batches(B, bias), Tq, Tk, words, s);
    if (*rc != RGD_OK) return nullptr;
    *room = tail;
    return words;
}

// measured: what a second and third resident workgroup add to a compute unit, and the duration of one inner
// step (64 keys or 64 query rows) of a workgroup that has its compute unit to itself
constexpr AttnSplitModel kFwdSplit = {1.3f, 1.5f, 0.9f};
constexpr AttnSplitModel kBwdSplit = {1.05f, 1.05f, 1.4f};

int check_common(const char* name, int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, int dtype, int bias_kind,
                 int bias_dtype, const rgd_tensor4* bias) {
    const int init_rc = rgd_attn_ready();
    if (init_rc != RGD_OK) return init_rc;
    RGD_REQUIRE(dtype == RGD_F16 || dtype == RGD_BF16, RGD_ERR_INVALID, "%s: Only support fp16 and bf16", name);
    RGD_REQUIRE(D >= 1 && D <= 128, RGD_ERR_INVALID, "%s: FlashAttention only support head dimensions up to 128", name);
    RGD_REQUIRE(B >= 0 && H >= 0 && Tq >= 0 && Tk >= 0, RGD_ERR_INVALID, "%s: negative shape", name);
    RGD_REQUIRE(Tq < (1ll << 30) && Tk < (1ll << 30) && B * H < (1ll << 24), RGD_ERR_UNSUPPORTED, "%s: shape too large",
                name);
    RGD_REQUIRE(bias_kind == RGD_BIAS_NONE || bias_kind == RGD_BIAS_VECTOR || bias_kind == RGD_BIAS_MATRIX,
                RGD_ERR_INVALID, "%s: bad bias kind %d", name, bias_kind);
    if (bias_kind != RGD_BIAS_NONE) {
        RGD_REQUIRE(bias && bias->ptr, RGD_ERR_INVALID, "%s: null bias", name);
        RGD_REQUIRE(bias_dtype == dtype || bias_dtype == RGD_F32, RGD_ERR_INVALID,
                    "%s: bias must have the dtype of q or fp32", name);
        // the kernels address a bias row block as a 32-bit lane offset: 16 rows plus a key index
        RGD_REQUIRE(bias_kind == RGD_BIAS_VECTOR || (bias->stride_n >= 0 && bias->stride_n < (int64_t(1) << 24)),
                    RGD_ERR_UNSUPPORTED,
                    "%s: bias row stride %lld is outside [0, 2^24)", name, (long long)bias->stride_n);
    }
    return RGD_OK;
}

}  // namespace

extern "C" {

int64_t rgd_attn_seqlen_q_rounded(int64_t Tq) { return (Tq + 63) / 64 * 64; }

size_t rgd_attn_fwd_workspace(int64_t B, int64_t, int64_t Tq, int64_t Tk, int64_t D) {
    if (D < 1 || D > 128) return 0;
    // two rounds of parts at the highest occupancy, then the tile classes of a head-shared bias
    const size_t cls = (D <= 64 && B > 0 && Tq > 0 && Tk > 0 && cls_nwords(Tk) <= CLS_MAX_WORDS && cls_nrow32(Tq) <= CLS_MAX_ROWS) ? cls_bytes(B, Tq, Tk) + 32 : 0;
    return (size_t)2 * rgd_num_cus() * 3 * fwd_part_bytes(attn_dpad(D)) + cls;
}

size_t rgd_attn_bias_classes_bytes(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* bias, int bias_kind,
                                   int bias_dtype) {
    if (B < 1 || !cls_eligible(H, Tq, Tk, D, bias, bias_kind, bias_dtype)) return 0;
    return cls_bytes(cls_batches(B, bias), Tq, Tk);
}

int rgd_attn_bias_classify(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* bias, int bias_kind,
                           int bias_dtype, void* classes, size_t classes_bytes, void* stream) {
    const char* name = "rgd_attn_bias_classify";
    const int init_rc = rgd_attn_ready();
    if (init_rc != RGD_OK) return init_rc;
    const size_t need = rgd_attn_bias_classes_bytes(B, H, Tq, Tk, D, bias, bias_kind, bias_dtype);
    RGD_REQUIRE(need > 0, RGD_ERR_UNSUPPORTED, "%s: no tile classes for this bias and shape (rgd_attn_bias_classes_bytes is 0)", name);
    RGD_REQUIRE(classes && (reinterpret_cast<uintptr_t>(classes) & 7u) == 0 && classes_bytes >= need, RGD_ERR_WORKSPACE,
                "%s: classes needs %zu bytes, 8-byte aligned", name, need);
    return attn_classify(bias->ptr, bias->stride_b, cls_row_stride(bias, bias_kind), bias_dtype, (int)cls_batches(B, bias), Tq, Tk,
                         static_cast<uint64_t*>(classes), static_cast<hipStream_t>(stream));
}

int rgd_attn_fwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* q, const rgd_tensor4* k,
                 const rgd_tensor4* v, const rgd_tensor4* bias, int bias_kind, int bias_dtype, const rgd_tensor4* o,
                 float* lse, int dtype, int causal, float softmax_scale, const void* bias_classes, void* workspace,
                 size_t workspace_bytes, void* stream) {
    const char* name = "rgd_attn_fwd";
    int rc = check_common(name, B, H, Tq, Tk, D, dtype, bias_kind, bias_dtype, bias);
    if (rc != RGD_OK) return rc;
    if (B * H * Tq == 0) return RGD_OK;
    RGD_REQUIRE(q && q->ptr && o && o->ptr && lse, RGD_ERR_INVALID, "%s: null tensor", name);
    RGD_REQUIRE(Tk == 0 || (k && k->ptr && v && v->ptr), RGD_ERR_INVALID, "%s: null tensor", name);

    // offsets inside one K/V tile are kept in 32 bits
    RGD_REQUIRE(Tk == 0 || (llabs(k->stride_n) < (1ll << 24) && llabs(v->stride_n) < (1ll << 24)), RGD_ERR_UNSUPPORTED,
                "%s: key/value token stride too large", name);

    AttnFwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = at(q);
    p.k = at(k);
    p.v = at(v);
    p.o = at(o);
    p.lse = lse;
    p.B = (int)B;
    p.H = (int)H;
    p.Tq = (int)Tq;
    p.Tk = (int)Tk;
    p.D = (int)D;
    p.Tq_rounded = (int)rgd_attn_seqlen_q_rounded(Tq);
    p.nqb = (int)((Tq + ATTN_BM - 1) / ATTN_BM);
    p.causal = causal ? 1 : 0;
    // (a bias matrix shared by the heads of a batch is also read once for four heads that way)
    const bool bias_shared = RGD_GROUP_SHARED_BIAS && bias_kind == RGD_BIAS_MATRIX && bias->stride_h == 0 && H % 4 == 0;
    p.group_lg = causal_group_lg(causal != 0 || bias_shared, B * H);
    p.vec = (D % 8 == 0) && t4_vec_ok(q) && (Tk == 0 || (t4_vec_ok(k) && t4_vec_ok(v))) && t4_vec_ok(o);
    p.scale_log2 = softmax_scale * kLog2e;
    p.bias_kind = bias_kind;
    p.bias_dtype = bias_dtype;
    if (bias_kind != RGD_BIAS_NONE) {
        p.bias = at(bias);
        if (bias_kind == RGD_BIAS_VECTOR) p.bias.sn = 0;
        const int64_t per16 = bias_dtype == RGD_F32 ? 4 : 8;  // elements per 16 bytes
        p.bias_vec = rgd_aligned16(bias->ptr) && (p.bias.sb % per16) == 0 && (p.bias.sh % per16) == 0 &&
                     (p.bias.sn % per16) == 0;
    }
    const int64_t items = (int64_t)p.nqb * B * H;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // tile classes of a head-shared bias: the caller's, or written into the end of the workspace
    size_t part_room = workspace_bytes;
    // (not with a softmax scale of 0 or below: the kernels that read classes add the bias in units of the raw scores)
    const void* cls = softmax_scale > 0.f ? cls_for_call(name, B, H, Tq, Tk, D, bias, bias_kind, bias_dtype, bias_classes, workspace,
                                                         workspace_bytes, 0, &part_room, s, &rc)
                                          : nullptr;
    if (rc != RGD_OK) return rc;
    if (cls) p.cls = cls_desc(cls, B, Tq, Tk, bias, bias_kind);
    // items of the last, partly filled round are split along the keys when a workspace is given
    const int dpad = attn_dpad(D);
    AttnSplit plan;
    if (workspace && rgd_aligned16(workspace) && !causal)
        plan = attn_split_plan(items, rgd_num_cus(), cls ? RGD_CLS_FWD_OCC : fwd_blocks_per_cu(dpad, bias_kind != RGD_BIAS_NONE),
                               (int)((Tk + ATTN_BN - 1) / ATTN_BN), fwd_part_bytes(dpad), part_room, kFwdSplit);
    p.split_full = plan.full;
    p.split_s = plan.s;
    // Leaving leading / trailing all -inf bias tiles out of a workgroup's loop takes a pass over its bias first.  It pays
    // when workgroups queue for compute units (the launch is then bound by the sum of their work); in a launch of one
    // round the time is that of the longest workgroup, which has no such tiles and only pays for the search.
    p.trim = items > (int64_t)rgd_num_cus() * fwd_blocks_per_cu(dpad, bias_kind != RGD_BIAS_NONE);
    if (plan.s > 1) {
        const size_t parts = (size_t)plan.items_split(items) * plan.s;
        p.part_o = static_cast<float*>(workspace);
        p.part_ml = p.part_o + parts * ATTN_BM * dpad;
    }
    const int64_t grid = plan.blocks(items);
    RGD_REQUIRE(grid < (1ll << 31), RGD_ERR_UNSUPPORTED, "%s: grid too large", name);
    if (cls) {
        // two launches over the same grid: batch elements whose bias is mostly ZERO / NEG tiles run in the variant laid
        // out like the kernel without bias, the others in the ordinary one (see cls_batch_dense)
        p.cls_take = 1;
        rc = dtype == RGD_F16 ? dispatch_fwd_cls<f16_t>(p, (unsigned)grid, s) : dispatch_fwd_cls<bf16_t>(p, (unsigned)grid, s);
        if (rc != RGD_OK) return rc;
        p.cls_take = 2;
    }
    rc = dtype == RGD_F16 ? dispatch_fwd<f16_t>(p, (unsigned)grid, s) : dispatch_fwd<bf16_t>(p, (unsigned)grid, s);
    if (rc != RGD_OK) return rc;
    if (plan.s > 1) {
        const unsigned n = (unsigned)plan.items_split(items);
        rc = dtype == RGD_F16 ? dispatch_fwd_merge<f16_t>(p, n, s) : dispatch_fwd_merge<bf16_t>(p, n, s);
        if (rc != RGD_OK) return rc;
        }
    return RGD_OK;
}

size_t rgd_attn_bwd_workspace(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, int mode) {
    // delta, dq_accum where the one-pass form may run, then room for two rounds of dK/dV parts (the dQ parts of the
    // two-kernel form reuse it; the launches are ordered)
    const int dpad = attn_dpad(D < 1 ? 1 : D);
    const bool accum = mode != RGD_ATTN_BWD_TWO_KERNEL && D <= 64 && (mode == RGD_ATTN_BWD_ONE_PASS || RGD_ATTN_BWD_AUTO_ONE_PASS);
    const size_t cls = (D <= 64 && B > 0 && Tq > 0 && Tk > 0 && cls_nwords(Tk) <= CLS_MAX_WORDS && cls_nrow32(Tq) <= CLS_MAX_ROWS)
                           ? cls_bytes(B, Tq, Tk) + 32
                           : 0;
    return bwd_delta_bytes(B, H, Tq) + (accum ? bwd_accum_bytes(B, H, Tq, dpad) : 0) +
           (size_t)2 * rgd_num_cus() * bwd_blocks_per_cu(dpad) * bwd_part_bytes(dpad, 2) + bwd_ranges_bytes(B, H, Tq, dpad) + 16 + cls;
}

int rgd_attn_bwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* dout, const rgd_tensor4* q,
                 const rgd_tensor4* k, const rgd_tensor4* v, const rgd_tensor4* o, const float* lse,
                 const rgd_tensor4* bias, int bias_kind, int bias_dtype, const rgd_tensor4* dq, const rgd_tensor4* dk,
                 const rgd_tensor4* dv, const rgd_tensor4* dbias, int dtype, int causal, float softmax_scale, int mode,
                 const void* bias_classes, void* workspace, size_t workspace_bytes, void* stream) {
    const char* name = "rgd_attn_bwd";
    RGD_REQUIRE(mode == RGD_ATTN_BWD_AUTO || mode == RGD_ATTN_BWD_TWO_KERNEL || mode == RGD_ATTN_BWD_ONE_PASS,
                RGD_ERR_INVALID, "%s: bad mode %d", name, mode);
    int rc = check_common(name, B, H, Tq, Tk, D, dtype, bias_kind, bias_dtype, bias);
    if (rc != RGD_OK) return rc;
    if (B * H == 0 || (Tq == 0 && Tk == 0)) return RGD_OK;
    const rgd_tensor4* all[] = {dout, q, k, v, o, dq, dk, dv};
    for (const rgd_tensor4* t : all) RGD_REQUIRE(t, RGD_ERR_INVALID, "%s: null tensor descriptor", name);
    RGD_REQUIRE(Tq == 0 || (dout->ptr && q->ptr && o->ptr && dq->ptr && lse), RGD_ERR_INVALID, "%s: null tensor", name);
    RGD_REQUIRE(Tk == 0 || (k->ptr && v->ptr && dk->ptr && dv->ptr), RGD_ERR_INVALID, "%s: null tensor", name);
    // offsets inside one staged tile (K, V in the dQ kernel; Q, dO in the dK/dV kernel) are kept in 32 bits
    for (const rgd_tensor4* t : {q, k, v, dout})
        RGD_REQUIRE(llabs(t->stride_n) < (1ll << 24), RGD_ERR_UNSUPPORTED, "%s: token stride %lld is outside (-2^24, 2^24)",
                    name, (long long)t->stride_n);
    // delta is required; whatever the workspace holds beyond it is used to split the last round of workgroups
    const size_t delta_bytes = bwd_delta_bytes(B, H, Tq);
    RGD_REQUIRE(workspace_bytes >= delta_bytes && (workspace || Tq == 0), RGD_ERR_WORKSPACE, "%s: workspace too small",
                name);
    const int dpad = attn_dpad(D);
    RGD_REQUIRE(mode != RGD_ATTN_BWD_ONE_PASS || D <= 64, RGD_ERR_UNSUPPORTED,
                "%s: the one-pass form covers head dims up to 64 (got %lld)", name, (long long)D);
    const bool want_dbias = dbias && dbias->ptr;
    if (want_dbias) {
        // written by the dQ kernel as 16-key runs of whole 64-key tiles: rows padded and 16-byte aligned
        const int64_t per16 = bias_dtype == RGD_F32 ? 4 : 8;
        RGD_REQUIRE(bias_kind != RGD_BIAS_NONE, RGD_ERR_INVALID, "%s: a bias gradient without a bias", name);
        RGD_REQUIRE(mode != RGD_ATTN_BWD_ONE_PASS, RGD_ERR_UNSUPPORTED,
                    "%s: the bias gradient comes from the dQ kernel of the two-kernel form", name);
        RGD_REQUIRE(dbias->stride_n >= (Tk + 63) / 64 * 64 && dbias->stride_n < (int64_t(1) << 31) &&
                        rgd_aligned16(dbias->ptr) && dbias->stride_b % per16 == 0 && dbias->stride_h % per16 == 0 &&
                        dbias->stride_n % per16 == 0,
                    RGD_ERR_INVALID, "%s: dbias needs 16-byte aligned rows of at least %lld elements (Tk rounded up to 64)",
                    name, (long long)((Tk + 63) / 64 * 64));
    }
    const size_t accum_bytes = bwd_accum_bytes(B, H, Tq, dpad);
    const bool one_pass = !want_dbias && bwd_one_pass(mode, D, workspace_bytes, delta_bytes + accum_bytes);
    RGD_REQUIRE(!one_pass || (workspace_bytes >= delta_bytes + accum_bytes && rgd_aligned16(workspace)), RGD_ERR_WORKSPACE,
                "%s: the one-pass form needs %zu bytes of 16-byte aligned workspace", name, delta_bytes + accum_bytes);
    const size_t fixed_bytes = delta_bytes + (one_pass ? accum_bytes : 0);
    const bool may_split = workspace && rgd_aligned16(workspace) && !causal;
    float* part_base = reinterpret_cast<float*>(static_cast<char*>(workspace) + fixed_bytes);
    size_t part_room = workspace_bytes - fixed_bytes;
    // With a bias at head dims above 64 the dQ launch notes, per 32 query rows, the keys whose bias is above -inf, and the
    // dK/dV launch starts every key block at the first rows that have such keys (a block-causal bias: half of its loop).
    // The notes live at the end of the workspace when it has room for them.
    int* ranges = nullptr;
    const size_t ranges_bytes = bwd_ranges_bytes(B, H, Tq, dpad);
    if (!one_pass && !want_dbias && !causal && bias_kind != RGD_BIAS_NONE && dpad > 64 && Tq > 0 && Tk > 0 && workspace &&
        workspace_bytes >= fixed_bytes + ranges_bytes + 16) {
        const size_t tail = (workspace_bytes - ranges_bytes) & ~(size_t)15;
        ranges = reinterpret_cast<int*>(static_cast<char*>(workspace) + tail);
        part_room = tail - fixed_bytes;
    }
    const int per_cu = one_pass ? RGD_FUSED_OCC : bwd_blocks_per_cu(dpad);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // tile classes of a head-shared bias (two-kernel form, no bias gradient): the caller's, or written into the end of
    // the workspace
    const void* cls = nullptr;
    if (!one_pass && !want_dbias && Tq > 0 && Tk > 0 && softmax_scale > 0.f) {
        size_t tail = workspace_bytes;
        cls = cls_for_call(name, B, H, Tq, Tk, D, bias, bias_kind, bias_dtype, bias_classes, workspace, workspace_bytes,
                           fixed_bytes, &tail, s, &rc);
        if (rc != RGD_OK) return rc;
        if (cls) part_room = tail - fixed_bytes;
    }

    AttnBwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = at(q);
    p.k = at(k);
    p.v = at(v);
    p.o = at(o);
    p.dout = at(dout);
    p.dq = at(dq);
    p.dk = at(dk);
    p.dv = at(dv);
    if (want_dbias) p.dbias = at(dbias);
    p.lse = lse;
    p.delta = static_cast<float*>(workspace);
    p.B = (int)B;
    p.H = (int)H;
    p.Tq = (int)Tq;
    p.Tk = (int)Tk;
    p.D = (int)D;
    p.Tq_rounded = (int)rgd_attn_seqlen_q_rounded(Tq);
    p.causal = causal ? 1 : 0;
    // (a bias matrix shared by the heads of a batch is also read once for four heads that way)
    const bool bias_shared = RGD_GROUP_SHARED_BIAS && bias_kind == RGD_BIAS_MATRIX && bias->stride_h == 0 && H % 4 == 0;
    p.group_lg = causal_group_lg(causal != 0 || bias_shared, B * H);
    p.vec = (D % 8 == 0);
    for (const rgd_tensor4* t : all) p.vec = p.vec && (t->ptr == nullptr || t4_vec_ok(t));
    p.scale = softmax_scale;
    p.scale_log2 = softmax_scale * kLog2e;
    p.bias_kind = bias_kind;
    p.bias_dtype = bias_dtype;
    if (bias_kind != RGD_BIAS_NONE) {
        p.bias = at(bias);
        if (bias_kind == RGD_BIAS_VECTOR) p.bias.sn = 0;
        const int64_t per16 = bias_dtype == RGD_F32 ? 4 : 8;
        p.bias_vec = rgd_aligned16(bias->ptr) && (p.bias.sb % per16) == 0 && (p.bias.sh % per16) == 0 &&
                     (p.bias.sn % per16) == 0;
    }
    if (cls) p.cls = cls_desc(cls, B, Tq, Tk, bias, bias_kind);
    if (one_pass) {
        p.dq_accum = reinterpret_cast<float*>(static_cast<char*>(workspace) + delta_bytes);
        if (Tq > 0) {  // delta, and dq_accum = 0
            rc = dtype == RGD_F16 ? dispatch_bwd_fused_aux<f16_t>(p, 0, s) : dispatch_bwd_fused_aux<bf16_t>(p, 0, s);
            if (rc != RGD_OK) return rc;
        }
        if (Tk > 0) {  // dK, dV and the dQ contributions of every key block
            p.nblk = (int)((Tk + BWD_BM - 1) / BWD_BM);
            const int64_t items = (int64_t)p.nblk * B * H;
            AttnSplit plan;
            if (may_split)
                plan = attn_split_plan(items, rgd_num_cus(), per_cu, (int)((Tq + 63) / 64), bwd_part_bytes(dpad, 2), part_room,
                                       kBwdSplit);
            p.split_full = plan.full;
            p.split_s = plan.s;
            p.part = part_base;
            const int64_t grid = plan.blocks(items);
            RGD_REQUIRE(grid < (1ll << 31), RGD_ERR_UNSUPPORTED, "%s: grid too large", name);
            rc = dtype == RGD_F16 ? dispatch_bwd_fused<f16_t>(p, (unsigned)grid, s) : dispatch_bwd_fused<bf16_t>(p, (unsigned)grid, s);
            if (rc != RGD_OK) return rc;
            if (plan.s > 1) {
                const unsigned n = (unsigned)plan.items_split(items);
                rc = dtype == RGD_F16 ? dispatch_bwd_merge<f16_t>(p, n, 2, s) : dispatch_bwd_merge<bf16_t>(p, n, 2, s);
                if (rc != RGD_OK) return rc;
            }
        }
        if (Tq > 0)  // dq = scale * dq_accum
            return dtype == RGD_F16 ? dispatch_bwd_fused_aux<f16_t>(p, 1, s) : dispatch_bwd_fused_aux<bf16_t>(p, 1, s);
        return RGD_OK;
    }
    if (Tq > 0) {  // dQ and delta
        p.nblk = (int)((Tq + BWD_BM - 1) / BWD_BM);
        const int64_t items = (int64_t)p.nblk * B * H;
        AttnSplit plan;
        if (may_split)
            plan = attn_split_plan(items, rgd_num_cus(), dq_blocks_per_cu(dpad), (int)((Tk + 63) / 64),
                                   bwd_part_bytes(dpad, 1), part_room, kBwdSplit);
        p.split_full = plan.full;
        p.split_s = plan.s;
        p.trim = items > (int64_t)rgd_num_cus() * dq_blocks_per_cu(dpad);  // see rgd_attn_fwd
        p.ranges = ranges;
        p.nrows32 = (int)bwd_rows32(Tq);
        p.part = part_base;
        const int64_t grid = plan.blocks(items);
        RGD_REQUIRE(grid < (1ll << 31), RGD_ERR_UNSUPPORTED, "%s: grid too large", name);
        if (cls) {  // two launches over the same grid, as in rgd_attn_fwd
            p.cls_take = 1;
            rc = dtype == RGD_F16 ? dispatch_bwd_cls<f16_t, true>(p, (unsigned)grid, s) : dispatch_bwd_cls<bf16_t, true>(p, (unsigned)grid, s);
            if (rc != RGD_OK) return rc;
            p.cls_take = 2;
        }
        rc = dtype == RGD_F16 ? dispatch_bwd<f16_t, true>(p, (unsigned)grid, s) : dispatch_bwd<bf16_t, true>(p, (unsigned)grid, s);
        if (rc != RGD_OK) return rc;
        if (plan.s > 1) {
            const unsigned n = (unsigned)plan.items_split(items);
            rc = dtype == RGD_F16 ? dispatch_bwd_merge<f16_t>(p, n, 1, s) : dispatch_bwd_merge<bf16_t>(p, n, 1, s);
            if (rc != RGD_OK) return rc;
        }
    }
    if (Tk > 0) {  // dK and dV (reads delta)
        p.nblk = (int)((Tk + BWD_BM - 1) / BWD_BM);
        const int64_t items = (int64_t)p.nblk * B * H;
        AttnSplit plan;
        if (may_split)
            plan = attn_split_plan(items, rgd_num_cus(), per_cu, (int)((Tq + 63) / 64), bwd_part_bytes(dpad, 2), part_room,
                                   kBwdSplit);
        p.split_full = plan.full;
        p.split_s = plan.s;
        p.trim = items > (int64_t)rgd_num_cus() * per_cu;
        p.ranges = ranges;
        p.nrows32 = (int)bwd_rows32(Tq);
        p.part = part_base;
        const int64_t grid = plan.blocks(items);
        RGD_REQUIRE(grid < (1ll << 31), RGD_ERR_UNSUPPORTED, "%s: grid too large", name);
        if (cls) {
            p.cls_take = 1;
            rc = dtype == RGD_F16 ? dispatch_bwd_cls<f16_t, false>(p, (unsigned)grid, s) : dispatch_bwd_cls<bf16_t, false>(p, (unsigned)grid, s);
            if (rc != RGD_OK) return rc;
            p.cls_take = 2;
        }
        rc = dtype == RGD_F16 ? dispatch_bwd<f16_t, false>(p, (unsigned)grid, s) : dispatch_bwd<bf16_t, false>(p, (unsigned)grid, s);
        if (rc != RGD_OK) return rc;
        if (plan.s > 1) {
            const unsigned n = (unsigned)plan.items_split(items);
            rc = dtype == RGD_F16 ? dispatch_bwd_merge<f16_t>(p, n, 2, s) : dispatch_bwd_merge<bf16_t>(p, n, 2, s);
            if (rc != RGD_OK) return rc;
        }
    }
    return RGD_OK;
}

}  // extern "C"
