// Row kernels for (B,T,C) tensors: RMSNorm and L2-normalize, forward and backward, over one or two
// tensors treated as one virtual tensor (blockIdx.x < nchunks of the first tensor selects it).
//
// Work decomposition: a row is owned by a group of G consecutive lanes; lane `lg` of the group holds
// the NV chunks [(k*G + lg)*VEC, +VEC), k < NV, in fp32 registers, so every element is read from
// HBM exactly once per pass (forward: x; backward: x and dy) and the row statistics never leave the
// wavefront.  rrms / rlen are recomputed in the backward from x, which is being read anyway.
//
// dw of RMSNorm: every lane accumulates xhat*dy for its own channels over the rows of the block;
// lanes, then waves, are combined in a fixed order into one fp32 partial row per block; partial rows
// are combined by a fan-in-16 tree in which the last block to arrive at a node (atomic ticket) adds
// the node's children in index order.  The result is independent of scheduling.
#pragma once

#include "common.h"

enum { WIDE_RMS = 0, WIDE_L2 = 1 };
constexpr int WIDE_FANIN = 16;
constexpr int WIDE_MAX_LEVELS = 5;

struct WideHalf {
    const void* x;
    const void* dy;
    void* y;  // forward output, or dx in the backward
    const void* w;
    void* dw;
    int64_t sx_b, sx_n, sd_b, sd_n, sy_b, sy_n, sw_b, sdw_b;
    int T, C, nchunks;
    int w_dtype, w_shared, w_vec;
    float inv_c;
    float* part;  // partial rows of every tree level
    int* ctr;     // arrival counters of every tree node (zero on entry, zero on exit)
    int nleaf;    // leaves per tree
    int tree_rows, tree_ctrs;
    int lvl_row_off[WIDE_MAX_LEVELS];
    int lvl_ctr_off[WIDE_MAX_LEVELS];
};

struct WideParams {
    WideHalf h[2];
    int rows_per_chunk;
    float eps;
};

template <typename T, int OP, bool BWD, int G, int NV, int VEC, bool VECTOR, int U, int NW>
__global__ __launch_bounds__(NW * 64) void wide_rows_kernel(const WideParams p) {
    extern __shared__ float s_dw[];
    __shared__ int s_last;

    const int which = (int)blockIdx.x >= p.h[0].nchunks ? 1 : 0;
    const WideHalf& h = p.h[which];
    const int chunk = blockIdx.x - (which ? p.h[0].nchunks : 0);
    const int b = blockIdx.y;
    const int C = h.C;
    const int r0 = chunk * p.rows_per_chunk;
    const int r1 = min(h.T, r0 + p.rows_per_chunk);

    constexpr int GPW = 64 / G;  // row groups per wave
    constexpr int NSLOT = NW * GPW;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int lg = lane % G;
    const int slot = wave * GPW + lane / G;

    const T* xb = static_cast<const T*>(h.x) + (int64_t)b * h.sx_b;
    const T* db = BWD ? static_cast<const T*>(h.dy) + (int64_t)b * h.sd_b : nullptr;
    T* yb = static_cast<T*>(h.y) + (int64_t)b * h.sy_b;

    constexpr bool HAS_W = (OP == WIDE_RMS);
    float wv[NV][VEC];
    float dwacc[NV][VEC];
    if constexpr (HAS_W) {
        const char* wp = static_cast<const char*>(h.w) + (int64_t)b * h.sw_b * (h.w_dtype == RGD_F32 ? 4 : 2);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (VECTOR && h.w_vec)
                load_chunk_dyn<VEC, VECTOR>(wp, h.w_dtype, (k * G + lg) * VEC, C, wv[k]);
            else
                load_chunk_dyn<VEC, false>(wp, h.w_dtype, (k * G + lg) * VEC, C, wv[k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) dwacc[k][e] = 0.f;
        }
    }

    for (int rbase = r0 + slot; rbase < r1; rbase += NSLOT * U) {
        float xv[U][NV][VEC];
        float dv[U][NV][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = rbase + u * NSLOT;
            const int lim = r < r1 ? C : 0;
            const T* xr = xb + (int64_t)r * h.sx_n;
#pragma unroll
            for (int k = 0; k < NV; ++k) load_chunk<T, VEC, VECTOR>(xr, (k * G + lg) * VEC, lim, xv[u][k]);
            if constexpr (BWD) {
                const T* dr = db + (int64_t)r * h.sd_n;
#pragma unroll
                for (int k = 0; k < NV; ++k) load_chunk<T, VEC, VECTOR>(dr, (k * G + lg) * VEC, lim, dv[u][k]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = rbase + u * NSLOT;
            const int lim = r < r1 ? C : 0;
            float ss = 0.f, sd = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float x = xv[u][k][e];
                    ss += x * x;
                    if constexpr (BWD) {
                        const float g = HAS_W ? dv[u][k][e] * wv[k][e] : dv[u][k][e];
                        sd += x * g;
                    }
                }
            ss = group_reduce<G>(ss);
            if constexpr (BWD) sd = group_reduce<G>(sd);
            float rn;  // rrms or rlen
            if constexpr (OP == WIDE_RMS) {
                rn = rsqrtf(ss * h.inv_c + p.eps);
            } else {
                const float len = sqrtf(ss);
                rn = len < p.eps ? 1.0f / p.eps : 1.0f / len;
            }
            float out[NV][VEC];
            if constexpr (!BWD) {
#pragma unroll
                for (int k = 0; k < NV; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        out[k][e] = HAS_W ? xv[u][k][e] * rn * wv[k][e] : xv[u][k][e] * rn;
            } else {
                // inner = mean(xhat*dy*w) for RMSNorm, sum(xhat*dy) for L2
                const float inner = OP == WIDE_RMS ? sd * rn * h.inv_c : sd * rn;
#pragma unroll
                for (int k = 0; k < NV; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float xh = xv[u][k][e] * rn;
                        const float g = HAS_W ? dv[u][k][e] * wv[k][e] : dv[u][k][e];
                        out[k][e] = (g - xh * inner) * rn;
                        if constexpr (HAS_W) dwacc[k][e] += xh * dv[u][k][e];
                    }
            }
            T* yr = yb + (int64_t)r * h.sy_n;
#pragma unroll
            for (int k = 0; k < NV; ++k) store_chunk<T, VEC, VECTOR>(yr, (k * G + lg) * VEC, lim, out[k]);
        }
    }

    if constexpr (BWD && HAS_W) {
        // ---- block partial: lanes that share channels, then waves, in a fixed order ----
#pragma unroll
        for (int k = 0; k < NV; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) dwacc[k][e] = cross_group_sum<G>(dwacc[k][e]);
        for (int wv_i = 0; wv_i < NW; ++wv_i) {
            if (wave == wv_i && lane < G) {
#pragma unroll
                for (int k = 0; k < NV; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const int c = (k * G + lg) * VEC + e;
                        if (c < C) s_dw[c] = wv_i == 0 ? dwacc[k][e] : s_dw[c] + dwacc[k][e];
                    }
            }
            __syncthreads();
        }

        const int tree = h.w_shared ? 0 : b;
        int idx = h.w_shared ? b * h.nchunks + chunk : chunk;
        int n = h.nleaf;
        void* dw_row = static_cast<char*>(h.dw) + (int64_t)tree * h.sdw_b * (h.w_dtype == RGD_F32 ? 4 : 2);
        if (n == 1) {
            for (int c = threadIdx.x; c < C; c += NW * 64) store_dyn(dw_row, h.w_dtype, c, s_dw[c]);
            return;
        }
        float* tree_part = h.part + (int64_t)tree * h.tree_rows * C;
        int* tree_ctr = h.ctr + (int64_t)tree * h.tree_ctrs;
        {
            float* mine = tree_part + (int64_t)(h.lvl_row_off[0] + idx) * C;
            for (int c = threadIdx.x; c < C; c += NW * 64) mine[c] = s_dw[c];
        }
        for (int lvl = 0;; ++lvl) {
            const int g = idx / WIDE_FANIN;
            const int gs = min(WIDE_FANIN, n - g * WIDE_FANIN);
            __threadfence();  // release this block's partial row
            __syncthreads();
            if (threadIdx.x == 0) {
                int* cp = tree_ctr + h.lvl_ctr_off[lvl] + g;
                const int t = __hip_atomic_fetch_add(cp, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
                const int last = (t == gs - 1);
                if (last) __hip_atomic_store(cp, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_last = last;
            }
            __syncthreads();
            if (!s_last) return;  // block-uniform
            __threadfence();      // acquire the siblings' rows
            const int ng = (n + WIDE_FANIN - 1) / WIDE_FANIN;
            const float* src = tree_part + (int64_t)(h.lvl_row_off[lvl] + g * WIDE_FANIN) * C;
            float* dst = tree_part + (int64_t)(h.lvl_row_off[lvl + 1] + g) * C;
            for (int c = threadIdx.x; c < C; c += NW * 64) {
                float acc = 0.f;
                for (int j = 0; j < gs; ++j)
                    acc += __hip_atomic_load(src + (int64_t)j * C + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (ng == 1)
                    store_dyn(dw_row, h.w_dtype, c, acc);
                else
                    dst[c] = acc;
            }
            if (ng == 1) return;
            idx = g;
            n = ng;
        }
    }
}

// host-side description of one (B,T,C) half handed to the launchers
struct WideHalfArgs {
    int64_t T = 0, C = 0;
    const rgd_tensor3* x = nullptr;
    const rgd_tensor3* dy = nullptr;
    const rgd_tensor3* y = nullptr;  // forward output or dx
    const rgd_tensor3* w = nullptr;
    const rgd_tensor3* dw = nullptr;
    int w_dtype = RGD_F32;
    int w_shared = 0;
};

int wide_launch(const char* name, int op, bool bwd, int64_t B, const WideHalfArgs& a1, const WideHalfArgs& a2,
                int dtype, float eps, void* workspace, size_t workspace_bytes, void* counters,
                size_t counter_bytes, void* stream);
int wide_workspace(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2, size_t* ws, size_t* ctr);

// per-dtype instantiation units (rows_wide_f32.hip, rows_wide_f16.hip, rows_wide_bf16.hip)
struct WideConfig {
    int op;
    bool bwd;
    int G, NV;
    bool vector;
};
// compile-time launch shape shared by the kernel instantiations and the host-side grid computation
constexpr int wide_unroll(bool bwd, int nv) { return bwd ? (nv == 1 ? 2 : 1) : (nv == 1 ? 4 : (nv == 2 ? 2 : 1)); }
constexpr int wide_waves(int op, bool bwd) { return (bwd && op == WIDE_RMS) ? 8 : 4; }
template <typename T> int wide_dispatch(const WideConfig& cfg, const WideParams& p, dim3 grid, size_t lds, hipStream_t s);
