// Host side of the per-head row kernels: validation, layout resolution, configuration choice and the
// extern "C" entry points for head LayerNorm, RoPE and LayerNorm+RoPE on (query, key).
#include "rows_head.h"

#include <algorithm>
#include <string.h>

namespace {

struct RopeArgs {
    const void* pe = nullptr;
    int64_t P = 0, R = 0, ss = 0, sn = 0;
    int dtype = RGD_F32;
    int64_t q_cutoff = 0, k_cutoff = 0;
    int bwd = 0;
};

bool t4_vec_ok(const rgd_tensor4* t, int es) {
    return rgd_aligned16(t->ptr) && (t->stride_b * es) % 16 == 0 && (t->stride_h * es) % 16 == 0 &&
           (t->stride_n * es) % 16 == 0;
}

int pow2ceil(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

void fill_strides(int64_t (&dst)[3], const rgd_tensor4* t, bool token_inner) {
    dst[0] = t->stride_b;
    dst[1] = token_inner ? t->stride_h : t->stride_n;
    dst[2] = token_inner ? t->stride_n : t->stride_h;
}

int head_launch(const char* name, int mode, int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D,
                const rgd_tensor4* xs[2], const rgd_tensor4* dys[2], const rgd_tensor4* ys[2], const RopeArgs* rope,
                int dtype, float eps, int max_d, void* stream) {
    rgd_ensure_init();
    RGD_REQUIRE(rgd_dtype_ok(dtype), RGD_ERR_INVALID, "%s: Only support fp16, bf16, and fp32", name);
    RGD_REQUIRE(B >= 0 && H >= 0 && Tq >= 0 && Tk >= 0 && D >= 1, RGD_ERR_INVALID, "%s: negative shape", name);
    RGD_REQUIRE(D <= max_d, RGD_ERR_INVALID, "%s: Only supports head dimensions up to %d", name, max_d);
    const bool bwd = mode == HEAD_LN_BWD || mode == HEAD_LNROPE_BWD;
    const int64_t T[2] = {Tq, Tk};
    const int64_t total = B * H * (Tq + Tk);
    RGD_REQUIRE(total < (1ll << 31), RGD_ERR_UNSUPPORTED, "%s: more than 2^31 rows", name);
    if (total == 0) return RGD_OK;
    const int es = rgd_dtype_size(dtype);

    HeadParams p;
    memset(&p, 0, sizeof(p));
    bool vector = (D * es) % 16 == 0;
    for (int i = 0; i < 2; ++i) {
        HeadHalf& h = p.h[i];
        if (B * H * T[i] == 0) {
            h.rows = 0;
            h.div12 = make_fastdiv(1);
            h.div2 = make_fastdiv(1);
            h.n12 = h.n2 = 1;
            continue;
        }
        RGD_REQUIRE(xs[i] && xs[i]->ptr && ys[i] && ys[i]->ptr && (!bwd || (dys[i] && dys[i]->ptr)), RGD_ERR_INVALID,
                    "%s: null tensor", name);
        // iterate rows in memory order: the index with the smaller stride is the inner one
        const bool token_inner = xs[i]->stride_n <= xs[i]->stride_h;
        const int64_t n1 = token_inner ? H : T[i];
        const int64_t n2 = token_inner ? T[i] : H;
        h.x = xs[i]->ptr;
        h.y = ys[i]->ptr;
        fill_strides(h.sx, xs[i], token_inner);
        fill_strides(h.sy, ys[i], token_inner);
        vector = vector && t4_vec_ok(xs[i], es) && t4_vec_ok(ys[i], es);
        if (bwd) {
            h.dy = dys[i]->ptr;
            fill_strides(h.sd, dys[i], token_inner);
            vector = vector && t4_vec_ok(dys[i], es);
        }
        h.rows = (uint32_t)(B * n1 * n2);
        h.n12 = (uint32_t)(n1 * n2);
        h.n2 = (uint32_t)n2;
        h.div12 = make_fastdiv(h.n12);
        h.div2 = make_fastdiv(h.n2);
        h.token_is_inner = token_inner ? 1 : 0;
        h.cutoff = 0;
    }
    p.D = (int)D;
    p.inv_d = 1.0f / (float)D;
    p.eps = eps;
    HeadConfig cfg;
    cfg.mode = mode;
    cfg.table_f32 = false;
    if (rope) {
        RGD_REQUIRE(rope->pe && rgd_dtype_ok(rope->dtype), RGD_ERR_INVALID, "%s: bad pos_emb", name);
        RGD_REQUIRE(rope->dtype == dtype || rope->dtype == RGD_F32, RGD_ERR_UNSUPPORTED,
                    "%s: pos_emb must have the dtype of the tensors or fp32", name);
        RGD_REQUIRE(rope->R >= 0 && rope->R <= D, RGD_ERR_INVALID, "%s: rotary dim %lld exceeds head dim %lld", name,
                    (long long)rope->R, (long long)D);
        RGD_REQUIRE(Tq < rope->P && Tk < rope->P, RGD_ERR_INVALID,
                    "%s: sequence length must be smaller than the pos_emb length %lld", name, (long long)rope->P);
        const int ps = rgd_dtype_size(rope->dtype);
        cfg.table_f32 = rope->dtype == RGD_F32 && dtype != RGD_F32;
        p.pe = rope->pe;
        p.pe_ss = rope->ss;
        p.pe_sn = rope->sn;
        p.R = (int)rope->R;
        p.rope_bwd = rope->bwd;
        p.h[0].cutoff = (int)std::max<int64_t>(0, std::min<int64_t>(rope->q_cutoff, Tq));
        p.h[1].cutoff = (int)std::max<int64_t>(0, std::min<int64_t>(rope->k_cutoff, Tk));
        if (rope->R == 0) {
            // nothing to rotate: the kernel still reads a table chunk per row and discards it, so point
            // the table at memory that certainly exists
            p.pe = xs[p.h[0].rows ? 0 : 1]->ptr;
            p.pe_ss = p.pe_sn = 0;
            cfg.table_f32 = false;
        } else {
            // the table is read with the same access width as the tensors
            const int vec_elems = 16 / es;
            vector = vector && rgd_aligned16(rope->pe) && (rope->ss * ps) % 16 == 0 && (rope->sn * ps) % 16 == 0 &&
                     (rope->R % vec_elems) == 0;
        }
    }

    cfg.vector = vector;
    // COMPACT addressing: every tensor's rows at one distance in iteration order, all byte offsets below 2^31
    bool compact = vector;
    const int64_t lim31 = (int64_t(1) << 31) - 64;
    for (int i = 0; i < 2 && compact; ++i) {
        HeadHalf& h = p.h[i];
        if (h.rows == 0) continue;
        const int64_t n2 = h.n2, n1 = h.n12 / h.n2;
        auto distance = [&](const int64_t* st, uint32_t* out) {
            const int64_t dist = n2 > 1 ? st[2] : (n1 > 1 ? st[1] : st[0]);
            // (row index and row distance below 2^24 each: the kernel multiplies them with the 24-bit multiplier)
            const bool ok = dist >= 0 && (n2 == 1 || st[2] == dist) && (n1 == 1 || st[1] == dist * n2) &&
                            (B == 1 || st[0] == dist * n1 * n2) && ((int64_t)h.rows * dist + D) * es < lim31 &&
                            h.rows < (1u << 24) && dist * es < (1 << 24);
            *out = ok ? (uint32_t)(dist * es) : 0u;
            return ok;
        };
        compact = distance(h.sx, &h.rbx) && distance(h.sy, &h.rby) && (!bwd || distance(h.sd, &h.rbd));
    }
    if (compact && rope) {
        const int64_t ps = rope->R == 0 ? 1 : rgd_dtype_size(rope->dtype);
        compact = p.pe_sn >= 0 && p.pe_ss >= 0 && rope->P < (1 << 24) && p.pe_sn * ps < (1 << 24) &&
                  (rope->P * p.pe_sn + D) * ps < lim31 && p.pe_ss * ps < lim31 &&
                  (rope->P * p.pe_sn + D) * ps + p.pe_ss * ps < lim31;
        p.pe_row_bytes = (uint32_t)(p.pe_sn * ps);
        p.pe_cos_bytes = (uint32_t)(p.pe_ss * ps);
    }
    cfg.compact = compact;
    const int vec = vector ? 16 / es : 2;
    const int chunks = (int)((D + vec - 1) / vec);
    if (chunks <= 64) {
        cfg.G = std::max(4, pow2ceil(chunks));
        cfg.NV = 1;
    } else {
        cfg.G = 64;
        cfg.NV = 2;
        RGD_REQUIRE(chunks <= 128, RGD_ERR_UNSUPPORTED, "%s: head dim too large", name);
    }
    const int rows_per_block = 4 * (64 / cfg.G) * head_unroll(mode, cfg.NV);
    p.blocks_q = (uint32_t)(((int64_t)p.h[0].rows + rows_per_block - 1) / rows_per_block);
    const int64_t blocks = p.blocks_q + ((int64_t)p.h[1].rows + rows_per_block - 1) / rows_per_block;
    p.nblocks = (uint32_t)blocks;
    const int64_t cap = RGD_HEAD_PERSIST > 0 ? (int64_t)rgd_num_cus() * RGD_HEAD_PERSIST : blocks;
    const dim3 grid((unsigned)std::min(blocks, cap), 1, 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc;
    if (dtype == RGD_F32)
        rc = head_dispatch<float>(cfg, p, grid, s);
    else if (dtype == RGD_F16)
        rc = head_dispatch<f16_t>(cfg, p, grid, s);
    else
        rc = head_dispatch<bf16_t>(cfg, p, grid, s);
    return rc;
}

}  // namespace

extern "C" {

int rgd_ln_qk_fwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* q, const rgd_tensor4* k,
                  const rgd_tensor4* qo, const rgd_tensor4* ko, int dtype, float eps, void* stream) {
    const rgd_tensor4* xs[2] = {q, k};
    const rgd_tensor4* ys[2] = {qo, ko};
    const rgd_tensor4* none[2] = {nullptr, nullptr};
    return head_launch("rgd_ln_qk_fwd", HEAD_LN_FWD, B, H, Tq, Tk, D, xs, none, ys, nullptr, dtype, eps, 256, stream);
}

int rgd_ln_qk_bwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* q, const rgd_tensor4* k,
                  const rgd_tensor4* dqo, const rgd_tensor4* dko, const rgd_tensor4* dq, const rgd_tensor4* dk,
                  int dtype, float eps, void* stream) {
    const rgd_tensor4* xs[2] = {q, k};
    const rgd_tensor4* ds[2] = {dqo, dko};
    const rgd_tensor4* ys[2] = {dq, dk};
    return head_launch("rgd_ln_qk_bwd", HEAD_LN_BWD, B, H, Tq, Tk, D, xs, ds, ys, nullptr, dtype, eps, 256, stream);
}

int rgd_rope_qk(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* q, const rgd_tensor4* k,
                const rgd_tensor4* qo, const rgd_tensor4* ko, const void* pos_emb, int64_t P, int64_t R,
                int64_t pe_stride_s, int64_t pe_stride_n, int pe_dtype, int64_t q_cutoff, int64_t k_cutoff, int is_bwd,
                int dtype, void* stream) {
    const rgd_tensor4* xs[2] = {q, k};
    const rgd_tensor4* ys[2] = {qo, ko};
    const rgd_tensor4* none[2] = {nullptr, nullptr};
    RopeArgs r;
    r.pe = pos_emb;
    r.P = P;
    r.R = R;
    r.ss = pe_stride_s;
    r.sn = pe_stride_n;
    r.dtype = pe_dtype;
    r.q_cutoff = q_cutoff;
    r.k_cutoff = k_cutoff;
    r.bwd = is_bwd ? 1 : 0;
    return head_launch("rgd_rope_qk", HEAD_ROPE, B, H, Tq, Tk, D, xs, none, ys, &r, dtype, 0.f, 128, stream);
}

int rgd_ln_rope_qk_fwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* q,
                       const rgd_tensor4* k, const rgd_tensor4* qo, const rgd_tensor4* ko, const void* pos_emb,
                       int64_t P, int64_t R, int64_t pe_stride_s, int64_t pe_stride_n, int pe_dtype, int64_t q_cutoff,
                       int64_t k_cutoff, int dtype, float eps, void* stream) {
    const rgd_tensor4* xs[2] = {q, k};
    const rgd_tensor4* ys[2] = {qo, ko};
    const rgd_tensor4* none[2] = {nullptr, nullptr};
    RopeArgs r;
    r.pe = pos_emb;
    r.P = P;
    r.R = R;
    r.ss = pe_stride_s;
    r.sn = pe_stride_n;
    r.dtype = pe_dtype;
    r.q_cutoff = q_cutoff;
    r.k_cutoff = k_cutoff;
    return head_launch("rgd_ln_rope_qk_fwd", HEAD_LNROPE_FWD, B, H, Tq, Tk, D, xs, none, ys, &r, dtype, eps, 128,
                       stream);
}

int rgd_ln_rope_qk_bwd(int64_t B, int64_t H, int64_t Tq, int64_t Tk, int64_t D, const rgd_tensor4* q,
                       const rgd_tensor4* k, const rgd_tensor4* dqo, const rgd_tensor4* dko, const rgd_tensor4* dq,
                       const rgd_tensor4* dk, const void* pos_emb, int64_t P, int64_t R, int64_t pe_stride_s,
                       int64_t pe_stride_n, int pe_dtype, int64_t q_cutoff, int64_t k_cutoff, int dtype, float eps,
                       void* stream) {
    const rgd_tensor4* xs[2] = {q, k};
    const rgd_tensor4* ds[2] = {dqo, dko};
    const rgd_tensor4* ys[2] = {dq, dk};
    RopeArgs r;
    r.pe = pos_emb;
    r.P = P;
    r.R = R;
    r.ss = pe_stride_s;
    r.sn = pe_stride_n;
    r.dtype = pe_dtype;
    r.q_cutoff = q_cutoff;
    r.k_cutoff = k_cutoff;
    r.bwd = 1;
    return head_launch("rgd_ln_rope_qk_bwd", HEAD_LNROPE_BWD, B, H, Tq, Tk, D, xs, ds, ys, &r, dtype, eps, 128, stream);
}

}  // extern "C"
