// Row kernels for per-head operators on query and key, (B,H,T,D) addressed by (b,h,n) strides:
// head LayerNorm (no affine), RoPE on the first R channels of the first `cutoff` tokens, and the
// fusion of the two, forward and backward.  q and k are one virtual tensor of rows: virtual row
// index < rows(q) selects q.
//
// A row (D <= 256 elements) is owned by G consecutive lanes; lane `lg` holds the NV chunks
// [(k*G + lg)*VEC, +VEC) in fp32 registers, so a wavefront works on 64/G rows at once and each
// tensor is read once.  VEC is even, so a rotary channel pair (2i, 2i+1) never straddles lanes.
// Mean and rstd are recomputed in the backward from the rows being read anyway.
//
// The body is straight-line code: every load of the U rows a lane group handles (inputs, upstream
// gradient, sin/cos rows) is issued unconditionally from a clamped address before anything is
// decoded, masks are applied with selects, and only the stores are predicated.
#pragma once

#include "common.h"

enum { HEAD_LN_FWD = 0, HEAD_LN_BWD = 1, HEAD_ROPE = 2, HEAD_LNROPE_FWD = 3, HEAD_LNROPE_BWD = 4 };

struct HeadHalf {
    const void* x;
    const void* dy;
    void* y;  // forward output, or dx
    int64_t sx[3], sd[3], sy[3];  // strides of (batch, outer index, inner index)
    uint32_t rows;                // B * N1 * N2
    FastDiv div12, div2;          // by N1*N2 and by N2
    uint32_t n12, n2;
    int token_is_inner;  // the inner index is the token (else the head)
    int cutoff;          // tokens >= cutoff are not rotated
    // COMPACT launches: the rows of x, dy and y lie at equal distances in iteration order (row r at r * bytes), and every
    // byte offset fits 31 bits
    uint32_t rbx, rbd, rby;
};

#ifndef RGD_HEAD_PERSIST
#define RGD_HEAD_PERSIST 32  // at most this many workgroups per compute unit, each walking several row blocks
// (measured on q,k (8,2048,16,64) bf16: 8 per unit lengthens the LN+RoPE step by 4 %, 16 by 1 %; 32, 64 and no cap are the same)
#endif
#ifndef RGD_HEAD_NT_STORE
#define RGD_HEAD_NT_STORE 0
#endif
struct HeadParams {
    HeadHalf h[2];
    uint32_t blocks_q;  // row blocks [0, blocks_q) belong to q, the rest to k
    uint32_t nblocks;   // row blocks in all; a workgroup takes blocks blockIdx.x, blockIdx.x + gridDim.x, ...
    int D;
    float inv_d, eps;
    const void* pe;  // (2, P, R) rotary table, [0] = sin, [1] = cos
    int64_t pe_ss, pe_sn;
    int R;
    int rope_bwd;  // flip the rotation sign
    uint32_t pe_row_bytes, pe_cos_bytes;  // COMPACT launches: bytes between table rows, and from the sin to the cos table
};

// T = tensor element type, TP = rotary table element type (T or float)
// FULL: D == G*NV*VEC, so no element of a lane's chunks is ever out of range
// COMPACT (with VECTOR and FULL): addresses are a uniform base plus a 32-bit byte offset per lane, row r of a tensor at
// r * its row distance.  The general form spends a quarter of its vector instructions on 64-bit address arithmetic
// (three 64-bit multiply-adds per tensor and row), and these kernels are bound by vector instruction issue as much as by
// memory: at 16 bytes per lane and row there are 160-240 instructions per row.
template <typename T, typename TP, int MODE, int G, int NV, int VEC, bool VECTOR, bool FULL, int U, bool COMPACT = false>
__global__ __launch_bounds__(256) void head_rows_kernel(const HeadParams p) {
    static_assert(!COMPACT || (VECTOR && FULL), "COMPACT: whole 16-byte chunks");
    constexpr bool HAS_LN = MODE != HEAD_ROPE;
    constexpr bool HAS_ROPE = MODE == HEAD_ROPE || MODE == HEAD_LNROPE_FWD || MODE == HEAD_LNROPE_BWD;
    constexpr bool BWD = MODE == HEAD_LN_BWD || MODE == HEAD_LNROPE_BWD;
    constexpr int GPW = 64 / G;
    constexpr int ROWS_PER_PASS = 4 * GPW;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int lg = lane % G;
    const int D = p.D;
    for (uint32_t vb = blockIdx.x; vb < p.nblocks; vb += gridDim.x) {
    const int which = vb >= p.blocks_q ? 1 : 0;  // block-uniform: scalar selects only
    const HeadHalf& h = p.h[which];
    const uint32_t row0 = (vb - (which ? p.blocks_q : 0u)) * (uint32_t)(ROWS_PER_PASS * U) + wave * GPW + lane / G;

    // x: plain (temporal) loads on purpose.  Non-temporal loads of x shorten the forward by 7 % but leave nothing
    // of q, k in the Infinity Cache for a backward that follows soon, which then takes 17 % longer; in the
    // backward they slow the next forward by a third.  dy is read once and nothing else wants it: non-temporal
    // (the forward+backward step gains 3 %).  Non-temporal stores change nothing.
    Chunk<T, VEC, VECTOR> xc[U][NV];
    Chunk<T, VEC, VECTOR, true> dc[U][NV];
    Chunk<TP, VEC, VECTOR> sc[U][NV], cc[U][NV];
    bool rotate[U];
    int lim[U];
    T* yrow[U];
    uint32_t yoff[U];  // COMPACT
    // COMPACT: this lane's bytes inside a row, and inside a table row (lanes past the rotary channels read its start)
    const uint32_t lane_bytes = (uint32_t)(lg * VEC) * (uint32_t)sizeof(T);
    const uint32_t lane_pe_bytes = (uint32_t)(lg * VEC < p.R ? lg * VEC : 0) * (uint32_t)sizeof(TP);

    // ---- phase 1: addresses and loads ----
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t r_raw = row0 + u * ROWS_PER_PASS;
        const bool valid = r_raw < h.rows;
        const uint32_t r = valid ? r_raw : h.rows - 1;  // a row that exists, result discarded
        const uint32_t b = fast_div(r, h.div12);
        const uint32_t rem = r - b * h.n12;
        const uint32_t i1 = fast_div(rem, h.div2);
        const uint32_t i2 = rem - i1 * h.n2;
        const int token = h.token_is_inner ? (int)i2 : (int)i1;
        lim[u] = valid ? D : 0;
        rotate[u] = HAS_ROPE && valid && token < h.cutoff;
        if constexpr (COMPACT) {
            constexpr uint32_t KSTEP = (uint32_t)(G * VEC) * (uint32_t)sizeof(T);
            const uint32_t xoff = __umul24(r, h.rbx) + lane_bytes;  // both below 2^24 (checked on the host)
            yoff[u] = __umul24(r, h.rby) + lane_bytes;
#pragma unroll
            for (int k = 0; k < NV; ++k) xc[u][k].load_at(h.x, xoff + k * KSTEP);
            if constexpr (BWD) {
                const uint32_t doff = __umul24(r, h.rbd) + lane_bytes;
#pragma unroll
                for (int k = 0; k < NV; ++k) dc[u][k].load_at(h.dy, doff + k * KSTEP);
            }
            if constexpr (HAS_ROPE) {
                const uint32_t poff = __umul24((uint32_t)token, p.pe_row_bytes) + lane_pe_bytes;
                const char* cos_base = static_cast<const char*>(p.pe) + p.pe_cos_bytes;
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    // chunk k of a lane starts at channel (k*G + lg)*VEC; past the rotary channels it reads the row's start
                    const uint32_t pk = (k == 0) ? poff
                                                 : __umul24((uint32_t)token, p.pe_row_bytes) +
                                                       (uint32_t)((k * G + lg) * VEC < p.R ? (k * G + lg) * VEC : 0) * (uint32_t)sizeof(TP);
                    sc[u][k].load_at(p.pe, pk);
                    cc[u][k].load_at(cos_base, pk);
                }
            }
        } else {
        const T* xr = static_cast<const T*>(h.x) + (int64_t)b * h.sx[0] + (int64_t)i1 * h.sx[1] + (int64_t)i2 * h.sx[2];
        yrow[u] = static_cast<T*>(h.y) + (int64_t)b * h.sy[0] + (int64_t)i1 * h.sy[1] + (int64_t)i2 * h.sy[2];
#pragma unroll
        for (int k = 0; k < NV; ++k) xc[u][k].load(xr, (k * G + lg) * VEC, D);
        if constexpr (BWD) {
            const T* dr = static_cast<const T*>(h.dy) + (int64_t)b * h.sd[0] + (int64_t)i1 * h.sd[1] + (int64_t)i2 * h.sd[2];
#pragma unroll
            for (int k = 0; k < NV; ++k) dc[u][k].load(dr, (k * G + lg) * VEC, D);
        }
        }
        if constexpr (HAS_ROPE && !COMPACT) {
            // token < T < P always holds, so the table row exists even for rows that are not rotated
            const TP* sin_row = static_cast<const TP*>(p.pe) + (int64_t)token * p.pe_sn;
            const TP* cos_row = sin_row + p.pe_ss;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                sc[u][k].load(sin_row, (k * G + lg) * VEC, p.R);
                cc[u][k].load(cos_row, (k * G + lg) * VEC, p.R);
            }
        }
    }

    // ---- phase 2: decode, transform, store ----
#pragma unroll
    for (int u = 0; u < U; ++u) {
        float xv[NV][VEC], dv[NV][VEC];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            xc[u][k].template decode<!FULL>((k * G + lg) * VEC, lim[u], xv[k]);
            if constexpr (BWD) dc[u][k].template decode<!FULL>((k * G + lg) * VEC, lim[u], dv[k]);
        }
        float rstd = 1.f;
        if constexpr (HAS_LN) {
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) s += xv[k][e];
            const float mean = group_reduce<G>(s) * p.inv_d;
            float ss = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xcen = (FULL || (k * G + lg) * VEC + e < lim[u]) ? xv[k][e] - mean : 0.f;
                    xv[k][e] = xcen;
                    ss += xcen * xcen;
                }
            rstd = rsqrtf(group_reduce<G>(ss) * p.inv_d + p.eps);
            // forward: xhat.  The backward keeps the centred x and folds rstd into its three row constants below
            // (two instructions per element less).
            if constexpr (!BWD) {
#pragma unroll
                for (int k = 0; k < NV; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) xv[k][e] *= rstd;
            }
        }
        if constexpr (HAS_ROPE) {
            // forward rotation (x0, x1) -> (-x1, x0); the backward uses (x1, -x0).  sin and cos are
            // taken at the output channel.  Applied to x in the forward modes, to dy in the backward.
            const bool flip = MODE == HEAD_ROPE ? p.rope_bwd != 0 : BWD;
            const int rlim = rotate[u] ? p.R : 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                float sn[VEC], cs[VEC];
                const int first = (k * G + lg) * VEC;
                sc[u][k].template decode<false>(first, rlim, sn);
                cc[u][k].template decode<false>(first, rlim, cs);
                float(&v)[VEC] = BWD ? dv[k] : xv[k];
                const float sgn = flip ? -1.f : 1.f;
#pragma unroll
                for (int e = 0; e < VEC; e += 2) {
                    const float x0 = v[e], x1 = v[e + 1];
                    const float o0 = x0 * cs[e] - sgn * x1 * sn[e];
                    const float o1 = x1 * cs[e + 1] + sgn * x0 * sn[e + 1];
                    // on the 16-byte path R is a multiple of the chunk, so a chunk rotates as a whole
                    v[e] = (VECTOR ? first < rlim : first + e < rlim) ? o0 : x0;
                    v[e + 1] = (VECTOR ? first < rlim : first + e + 1 < rlim) ? o1 : x1;
                }
            }
        }
        float out[NV][VEC];
        if constexpr (!BWD) {
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) out[k][e] = xv[k][e];
        } else {
            float si = 0.f, sg = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    si += xv[k][e] * dv[k][e];
                    sg += dv[k][e];
                }
            // dx = (dy - xhat * mean(xhat dy) - mean(dy)) * rstd with xhat = xc * rstd (xc = x - mean, what xv holds):
            //    = dy * rstd - xc * (rstd^3 mean(xc dy)) - mean(dy) * rstd
            const float inner = group_reduce<G>(si) * p.inv_d;  // mean(xc dy)
            const float mdy = group_reduce<G>(sg) * p.inv_d;
            const float cx = -(rstd * rstd) * (rstd * inner), c0 = -mdy * rstd;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) out[k][e] = fmaf(xv[k][e], cx, fmaf(dv[k][e], rstd, c0));
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if constexpr (COMPACT)
                store_chunk_at<T, VEC, RGD_HEAD_NT_STORE != 0>(h.y, yoff[u] + k * (uint32_t)(G * VEC * sizeof(T)), lim[u] != 0, out[k]);
            else
                store_chunk<T, VEC, VECTOR, RGD_HEAD_NT_STORE != 0>(yrow[u], (k * G + lg) * VEC, lim[u], out[k]);
        }
    }
    }  // row blocks of this workgroup
}

struct HeadConfig {
    int mode;
    int G, NV;
    bool vector;
    bool compact;    // rows at equal distances, 31-bit byte offsets (see head_rows_kernel)
    bool table_f32;  // rotary table is fp32 while the tensors are 16-bit
};
#ifndef RGD_HEAD_U_FWD
#define RGD_HEAD_U_FWD 4
#endif
#ifndef RGD_HEAD_U_BWD
#define RGD_HEAD_U_BWD 2
#endif
constexpr int head_unroll(int mode, int nv) {
    return nv > 1 ? 1 : ((mode == HEAD_LN_BWD || mode == HEAD_LNROPE_BWD) ? RGD_HEAD_U_BWD : RGD_HEAD_U_FWD);
}
template <typename T> int head_dispatch(const HeadConfig& cfg, const HeadParams& p, dim3 grid, hipStream_t s);
