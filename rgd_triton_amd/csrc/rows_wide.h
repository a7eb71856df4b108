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

// WPR = wavefronts per row.  1: a row is owned by G <= 64 lanes of one wavefront.  4: a row is owned by
// all 256 lanes of 4 wavefronts (G == 64), the row statistics are combined through LDS; used for rows
// too wide to keep x, dy, w and the dw accumulators of one row in the registers of 64 lanes.
template <typename T, int OP, bool BWD, int G, int NV, int VEC, bool VECTOR, int U, int NW, int WPR>
__global__ __launch_bounds__(NW * 64) void wide_rows_kernel(const WideParams p) {
    extern __shared__ float s_dw[];
    __shared__ int s_last;
    __shared__ float s_red[2][2][NW];  // [parity][statistic][wavefront]
    static_assert(WPR == 1 || G == 64, "multi-wavefront rows use whole wavefronts");

    const int which = (int)blockIdx.x >= p.h[0].nchunks ? 1 : 0;
    const WideHalf& h = p.h[which];
    const int chunk = blockIdx.x - (which ? p.h[0].nchunks : 0);
    const int b = blockIdx.y;
    const int C = h.C;
    const int r0 = chunk * p.rows_per_chunk;
    const int r1 = min(h.T, r0 + p.rows_per_chunk);

    constexpr int GPW = 64 / G;               // rows per wavefront at a time (WPR == 1)
    constexpr int NSLOT = NW * GPW / WPR;     // rows the block works on at a time
    constexpr int GL = G * WPR;               // lanes per row
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int wsub = wave % WPR;              // position of this wavefront inside its row group
    const int lg = wsub * 64 + lane % G;      // lane index inside the row
    const int slot = WPR == 1 ? wave * GPW + lane / G : wave / WPR;

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
                load_chunk_dyn<VEC, VECTOR>(wp, h.w_dtype, (k * GL + lg) * VEC, C, wv[k]);
            else
                load_chunk_dyn<VEC, false>(wp, h.w_dtype, (k * GL + lg) * VEC, C, wv[k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) dwacc[k][e] = 0.f;
        }
    }

    // the trip count is the same for every wavefront of the block (rows past the end are masked), so the
    // block-wide barriers of the multi-wavefront mode are reached by everyone
    const int iters = (r1 - r0 + NSLOT * U - 1) / (NSLOT * U);
    for (int it = 0; it < iters; ++it) {
        const int rbase = r0 + slot + it * NSLOT * U;
        Chunk<T, VEC, VECTOR> xc[U][NV], dc[U][NV];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = min(rbase + u * NSLOT, r1 - 1);  // a row that exists; masked below if past the end
            const T* xr = xb + (int64_t)r * h.sx_n;
#pragma unroll
            for (int k = 0; k < NV; ++k) xc[u][k].load(xr, (k * GL + lg) * VEC, C);
            if constexpr (BWD) {
                const T* dr = db + (int64_t)r * h.sd_n;
#pragma unroll
                for (int k = 0; k < NV; ++k) dc[u][k].load(dr, (k * GL + lg) * VEC, C);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = rbase + u * NSLOT;
            const int lim = r < r1 ? C : 0;
            float xv[NV][VEC], dv[NV][VEC];
            float ss = 0.f, sd = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                xc[u][k].decode((k * GL + lg) * VEC, lim, xv[k]);
                if constexpr (BWD) dc[u][k].decode((k * GL + lg) * VEC, lim, dv[k]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float x = xv[k][e];
                    ss += x * x;
                    if constexpr (BWD) {
                        const float gr = HAS_W ? dv[k][e] * wv[k][e] : dv[k][e];
                        sd += x * gr;
                    }
                }
            }
            ss = group_reduce<G>(ss);
            if constexpr (BWD) sd = group_reduce<G>(sd);
            if constexpr (WPR > 1) {
                const int par = (it * U + u) & 1;
                if (lane == 0) {
                    s_red[par][0][wave] = ss;
                    if constexpr (BWD) s_red[par][1][wave] = sd;
                }
                __syncthreads();
                const int w0 = wave - wsub;
                ss = 0.f;
                sd = 0.f;
#pragma unroll
                for (int i = 0; i < WPR; ++i) {
                    ss += s_red[par][0][w0 + i];
                    if constexpr (BWD) sd += s_red[par][1][w0 + i];
                }
            }
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
                    for (int e = 0; e < VEC; ++e) out[k][e] = HAS_W ? xv[k][e] * rn * wv[k][e] : xv[k][e] * rn;
            } else {
                // inner = mean(xhat*dy*w) for RMSNorm, sum(xhat*dy) for L2
                const float inner = OP == WIDE_RMS ? sd * rn * h.inv_c : sd * rn;
#pragma unroll
                for (int k = 0; k < NV; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float xh = xv[k][e] * rn;
                        const float gr = HAS_W ? dv[k][e] * wv[k][e] : dv[k][e];
                        out[k][e] = (gr - xh * inner) * rn;
                        if constexpr (HAS_W) dwacc[k][e] += xh * dv[k][e];
                    }
            }
            T* yr = yb + (int64_t)min(r, r1 - 1) * h.sy_n;
#pragma unroll
            for (int k = 0; k < NV; ++k) store_chunk<T, VEC, VECTOR>(yr, (k * GL + lg) * VEC, lim, out[k]);
        }
    }

    if constexpr (BWD && HAS_W) {
        // ---- block partial: lanes that share channels, then waves, in a fixed order ----
#pragma unroll
        for (int k = 0; k < NV; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) dwacc[k][e] = cross_group_sum<G>(dwacc[k][e]);
        // wavefront w covers the channels of row position (w % WPR); the first WPR wavefronts store, the
        // others add, one wavefront at a time
        for (int wv_i = 0; wv_i < NW; ++wv_i) {
            if (wave == wv_i && lane < G) {
#pragma unroll
                for (int k = 0; k < NV; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const int c = (k * GL + lg) * VEC + e;
                        if (c < C) s_dw[c] = wv_i < WPR ? dwacc[k][e] : s_dw[c] + dwacc[k][e];
                    }
            }
            if (wv_i % WPR == WPR - 1) __syncthreads();
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
        // Partial rows travel between blocks through agent-scope (write-through) stores and loads, and
        // each block waits for its own stores to complete before it takes a ticket.  That is all the
        // ordering the tree needs, and it avoids a release fence, which on this multi-XCD part would
        // write back the whole L2 (full of freshly written dx) once per block.
        {
            float* mine = tree_part + (int64_t)(h.lvl_row_off[0] + idx) * C;
            for (int c = threadIdx.x; c < C; c += NW * 64)
                __hip_atomic_store(mine + c, s_dw[c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        for (int lvl = 0;; ++lvl) {
            const int g = idx / WIDE_FANIN;
            const int gs = min(WIDE_FANIN, n - g * WIDE_FANIN);
            __builtin_amdgcn_s_waitcnt(0);  // this thread's partial-row stores have completed
            __syncthreads();
            if (threadIdx.x == 0) {
                int* cp = tree_ctr + h.lvl_ctr_off[lvl] + g;
                const int t = __hip_atomic_fetch_add(cp, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const int last = (t == gs - 1);
                if (last) __hip_atomic_store(cp, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_last = last;
            }
            __syncthreads();
            if (!s_last) return;  // block-uniform
            const int ng = (n + WIDE_FANIN - 1) / WIDE_FANIN;
            const float* src = tree_part + (int64_t)(h.lvl_row_off[lvl] + g * WIDE_FANIN) * C;
            float* dst = tree_part + (int64_t)(h.lvl_row_off[lvl + 1] + g) * C;
            for (int c = threadIdx.x; c < C; c += NW * 64) {
                float v[WIDE_FANIN];
#pragma unroll
                for (int j = 0; j < WIDE_FANIN; ++j)
                    v[j] = j < gs ? __hip_atomic_load(src + (int64_t)j * C + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                  : 0.f;
                float acc = 0.f;
#pragma unroll
                for (int j = 0; j < WIDE_FANIN; ++j) acc += v[j];  // fixed order
                if (ng == 1)
                    store_dyn(dw_row, h.w_dtype, c, acc);
                else
                    __hip_atomic_store(dst + c, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
    int G, NV, WPR;
    bool vector;
};
// compile-time launch shape shared by the kernel instantiations and the host-side grid computation
constexpr int wide_unroll(bool bwd, int nv) { return bwd ? (nv == 1 ? 2 : 1) : (nv == 1 ? 4 : (nv == 2 ? 2 : 1)); }
constexpr int wide_waves(int op, bool bwd) { return (bwd && op == WIDE_RMS) ? 8 : 4; }
template <typename T> int wide_dispatch(const WideConfig& cfg, const WideParams& p, dim3 grid, size_t lds, hipStream_t s);
