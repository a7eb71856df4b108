// Row kernels for per-head operators on query and key, (B,H,T,D) addressed by (b,h,n) strides:
// head LayerNorm (no affine), RoPE on the first R channels of the first `cutoff` tokens, and the
// fusion of the two, forward and backward.  q and k are one virtual tensor of rows: virtual row
// index < rows(q) selects q.
//
// A row (D <= 256 elements) is owned by G consecutive lanes; lane `lg` holds the NV chunks
// [(k*G + lg)*VEC, +VEC) in fp32 registers, so a wavefront works on 64/G rows at once and each
// tensor is read once.  VEC is even, so a rotary channel pair (2i, 2i+1) never straddles lanes.
// Mean and rstd are recomputed in the backward from the rows being read anyway.
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
};

struct HeadParams {
    HeadHalf h[2];
    uint32_t total_rows;
    int D;
    float inv_d, eps;
    const void* pe;  // (2, P, R) rotary table, [0] = sin, [1] = cos
    int64_t pe_ss, pe_sn;
    int pe_dtype, pe_vec, R;
    int rope_bwd;  // flip the rotation sign
};

template <int NV, int VEC, int G, bool VECTOR>
__device__ __forceinline__ void rope_apply(float (&v)[NV][VEC], const HeadParams& p, int token, int lg, bool bwd) {
    const int esz = p.pe_dtype == RGD_F32 ? 4 : 2;
    const char* sin_row = static_cast<const char*>(p.pe) + (int64_t)token * p.pe_sn * esz;
    const char* cos_row = sin_row + p.pe_ss * esz;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int first = (k * G + lg) * VEC;
        if (first < p.R) {
            float sn[VEC], cs[VEC];
            if (VECTOR && p.pe_vec) {
                load_chunk_dyn<VEC, VECTOR>(sin_row, p.pe_dtype, first, p.R, sn);
                load_chunk_dyn<VEC, VECTOR>(cos_row, p.pe_dtype, first, p.R, cs);
            } else {
                load_chunk_dyn<VEC, false>(sin_row, p.pe_dtype, first, p.R, sn);
                load_chunk_dyn<VEC, false>(cos_row, p.pe_dtype, first, p.R, cs);
            }
#pragma unroll
            for (int e = 0; e < VEC; e += 2) {
                const float x0 = v[k][e], x1 = v[k][e + 1];
                // forward rotation (x0, x1) -> (-x1, x0); the backward uses (x1, -x0).  sin and cos
                // are taken at the output channel.
                const float r0 = bwd ? x1 : -x1;
                const float r1 = bwd ? -x0 : x0;
                if (first + e < p.R) v[k][e] = x0 * cs[e] + r0 * sn[e];
                if (first + e + 1 < p.R) v[k][e + 1] = x1 * cs[e + 1] + r1 * sn[e + 1];
            }
        }
    }
}

template <typename T, int MODE, int G, int NV, int VEC, bool VECTOR, int U>
__global__ __launch_bounds__(256) void head_rows_kernel(const HeadParams p) {
    constexpr bool HAS_LN = MODE != HEAD_ROPE;
    constexpr bool HAS_ROPE = MODE == HEAD_ROPE || MODE == HEAD_LNROPE_FWD || MODE == HEAD_LNROPE_BWD;
    constexpr bool BWD = MODE == HEAD_LN_BWD || MODE == HEAD_LNROPE_BWD;
    constexpr int GPW = 64 / G;
    constexpr int ROWS_PER_PASS = 4 * GPW;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int lg = lane % G;
    const uint32_t row0 = blockIdx.x * (uint32_t)(ROWS_PER_PASS * U) + wave * GPW + lane / G;
    const int D = p.D;

    float xv[U][NV][VEC];
    float dv[U][NV][VEC];
    int token[U];
    int cut[U];
    int lim[U];
    T* yrow[U];

#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t vr = row0 + u * ROWS_PER_PASS;
        const bool valid = vr < p.total_rows;
        const int which = (valid && vr >= p.h[0].rows) ? 1 : 0;
        const HeadHalf& h = p.h[which];
        const uint32_t r = valid ? vr - (which ? p.h[0].rows : 0u) : 0u;
        const uint32_t b = fast_div(r, h.div12);
        const uint32_t rem = r - b * h.n12;
        const uint32_t i1 = fast_div(rem, h.div2);
        const uint32_t i2 = rem - i1 * h.n2;
        token[u] = h.token_is_inner ? (int)i2 : (int)i1;
        cut[u] = h.cutoff;
        lim[u] = valid ? D : 0;
        const T* xr = static_cast<const T*>(h.x) + (int64_t)b * h.sx[0] + (int64_t)i1 * h.sx[1] + (int64_t)i2 * h.sx[2];
        yrow[u] = static_cast<T*>(h.y) + (int64_t)b * h.sy[0] + (int64_t)i1 * h.sy[1] + (int64_t)i2 * h.sy[2];
#pragma unroll
        for (int k = 0; k < NV; ++k) load_chunk<T, VEC, VECTOR>(xr, (k * G + lg) * VEC, lim[u], xv[u][k]);
        if constexpr (BWD) {
            const T* dr = static_cast<const T*>(h.dy) + (int64_t)b * h.sd[0] + (int64_t)i1 * h.sd[1] + (int64_t)i2 * h.sd[2];
#pragma unroll
            for (int k = 0; k < NV; ++k) load_chunk<T, VEC, VECTOR>(dr, (k * G + lg) * VEC, lim[u], dv[u][k]);
        }
    }

#pragma unroll
    for (int u = 0; u < U; ++u) {
        float rstd = 1.f;
        if constexpr (HAS_LN) {
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) s += xv[u][k][e];
            const float mean = group_reduce<G>(s) * p.inv_d;
            float ss = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xc = ((k * G + lg) * VEC + e < lim[u]) ? xv[u][k][e] - mean : 0.f;
                    xv[u][k][e] = xc;
                    ss += xc * xc;
                }
            rstd = rsqrtf(group_reduce<G>(ss) * p.inv_d + p.eps);
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) xv[u][k][e] *= rstd;  // xhat
        }
        const bool rotate = HAS_ROPE && lim[u] != 0 && token[u] < cut[u];
        if constexpr (!BWD) {
            if constexpr (HAS_ROPE) {
                if (rotate) rope_apply<NV, VEC, G, VECTOR>(xv[u], p, token[u], lg, MODE == HEAD_ROPE ? p.rope_bwd != 0 : false);
            }
#pragma unroll
            for (int k = 0; k < NV; ++k) store_chunk<T, VEC, VECTOR>(yrow[u], (k * G + lg) * VEC, lim[u], xv[u][k]);
        } else {
            if constexpr (HAS_ROPE) {
                if (rotate) rope_apply<NV, VEC, G, VECTOR>(dv[u], p, token[u], lg, true);
            }
            float si = 0.f, sg = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    si += xv[u][k][e] * dv[u][k][e];
                    sg += dv[u][k][e];
                }
            const float inner = group_reduce<G>(si) * p.inv_d;
            const float mdy = group_reduce<G>(sg) * p.inv_d;
            float out[NV][VEC];
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) out[k][e] = (dv[u][k][e] - xv[u][k][e] * inner - mdy) * rstd;
#pragma unroll
            for (int k = 0; k < NV; ++k) store_chunk<T, VEC, VECTOR>(yrow[u], (k * G + lg) * VEC, lim[u], out[k]);
        }
    }
}

struct HeadConfig {
    int mode;
    int G, NV;
    bool vector;
};
constexpr int head_unroll(int mode, int nv) {
    return nv > 1 ? 1 : ((mode == HEAD_LN_BWD || mode == HEAD_LNROPE_BWD) ? 2 : 4);
}
template <typename T> int head_dispatch(const HeadConfig& cfg, const HeadParams& p, dim3 grid, hipStream_t s);
