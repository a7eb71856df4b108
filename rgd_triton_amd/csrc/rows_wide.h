// Row kernels for (B,T,C) tensors: RMSNorm and L2-normalize, forward and backward, over one or two
// tensors treated as one virtual tensor (blockIdx.x < nchunks of the first tensor selects it).
//
// Work decomposition: a row is owned by a group of G consecutive lanes; lane `lg` of the group holds
// the NV chunks [(k*G + lg)*VEC, +VEC), k < NV, in fp32 registers, so every element is read from
// HBM exactly once per pass (forward: x; backward: x and dy) and the row statistics never leave the
// wavefront.  rrms / rlen are recomputed in the backward from x, which is being read anyway.
//
// dw of RMSNorm: every lane accumulates xhat*dy for its own channels over the rows of the block;
// lanes, then waves, are combined in a fixed order into one fp32 partial row per block.  A second, small
// kernel (wide_dw_reduce_kernel) adds the partial rows of a weight in a fixed order.  The result is
// independent of scheduling.  (Combining the rows inside the first kernel, with arrival tickets, was
// measured slower: every level of such a tree costs several microseconds of cross-XCD round trips.)
#pragma once

#include <type_traits>
#ifndef RGD_WIDE_RMS_FWD_64
#define RGD_WIDE_RMS_FWD_64 1
#endif

#include "common.h"

enum { WIDE_RMS = 0, WIDE_L2 = 1 };
#ifndef RGD_WIDE_EPL_U2
#define RGD_WIDE_EPL_U2 16  // backward: two rows in flight up to this many elements per lane
#endif
#ifndef RGD_WIDE_RED_WAVES
#define RGD_WIDE_RED_WAVES 16
#endif
constexpr int WIDE_RED_WAVES = RGD_WIDE_RED_WAVES;  // wavefronts of a reduce block; wavefront w adds partial rows w, w+WAVES, ...

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
    float* part;  // (weights, nleaf, C) partial rows, one per block
    int nleaf;    // partial rows per weight
    int red_blocks;  // reduce-kernel blocks of this half: weights * ceil(C / 64)
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
    extern __shared__ __attribute__((aligned(16))) float s_dw[];  // backward with weights: NW/WPR rows of C sums
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
        // The weight's element type and alignment are known at run time only.  One decision for the whole row, and inside
        // it all NV chunk loads go out before the first is decoded: one round trip to memory in front of the row loop
        // instead of NV of them (a kernel of the small configurations lasts a handful of such round trips).
        auto load_w = [&](auto tag, auto vec_ok) __attribute__((always_inline)) {
            typedef decltype(tag) TW;
            constexpr bool V = decltype(vec_ok)::value;
            Chunk<TW, VEC, V> wc[NV];
#pragma unroll
            for (int k = 0; k < NV; ++k) wc[k].load(reinterpret_cast<const TW*>(wp), (k * GL + lg) * VEC, C);
#pragma unroll
            for (int k = 0; k < NV; ++k) wc[k].template decode<true>((k * GL + lg) * VEC, C, wv[k]);
        };
        if (VECTOR && h.w_vec) {
            if (h.w_dtype == RGD_BF16) load_w(bf16_t{}, std::integral_constant<bool, VECTOR>{});
            else if (h.w_dtype == RGD_F16) load_w(f16_t{}, std::integral_constant<bool, VECTOR>{});
            else load_w(float{}, std::integral_constant<bool, VECTOR>{});
        } else {
            if (h.w_dtype == RGD_BF16) load_w(bf16_t{}, std::false_type{});
            else if (h.w_dtype == RGD_F16) load_w(f16_t{}, std::false_type{});
            else load_w(float{}, std::false_type{});
        }
#pragma unroll
        for (int k = 0; k < NV; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) dwacc[k][e] = 0.f;
    }

    // the trip count is the same for every wavefront of the block (rows past the end are masked), so the
    // block-wide barriers of the multi-wavefront mode are reached by everyone
    const int iters = (r1 - r0 + NSLOT * U - 1) / (NSLOT * U);
    for (int it = 0; it < iters; ++it) {
        const int rbase = r0 + slot + it * NSLOT * U;
        Chunk<T, VEC, VECTOR, !BWD> xc[U][NV];  // forward: x is read with non-temporal loads
        Chunk<T, VEC, VECTOR, true> dc[U][NV];   // the upstream gradient is read once: non-temporal
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
        // ---- block partial: lanes that share channels, then the wavefronts' rows, in a fixed order ----
#pragma unroll
        for (int k = 0; k < NV; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) dwacc[k][e] = cross_group_sum<G>(dwacc[k][e]);
        // every wavefront (every group of WPR wavefronts) leaves its sums in an LDS row of its own, all at
        // once; then each thread adds the rows for a few channels in row order
        constexpr int NR = NW / WPR;
        float* my_row = s_dw + (wave / WPR) * C;
        if (lane < G) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int c0 = (k * GL + lg) * VEC;
                if (VECTOR && VEC % 4 == 0 && (C & 3) == 0) {  // C % 4 == 0: chunks are whole and 16-byte aligned
                    if (c0 < C) {
#pragma unroll
                        for (int e = 0; e < VEC; e += 4)
                            *reinterpret_cast<f32x4*>(my_row + c0 + e) =
                                f32x4{dwacc[k][e], dwacc[k][e + 1], dwacc[k][e + 2], dwacc[k][e + 3]};
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        if (c0 + e < C) my_row[c0 + e] = dwacc[k][e];
                }
            }
        }
        __syncthreads();

        const int wgt = h.w_shared ? 0 : b;  // which weight this block contributes to
        const int idx = h.w_shared ? b * h.nchunks + chunk : chunk;
        void* dw_row = static_cast<char*>(h.dw) + (int64_t)wgt * h.sdw_b * (h.w_dtype == RGD_F32 ? 4 : 2);
        float* mine = h.part + ((int64_t)wgt * h.nleaf + idx) * C;
        for (int c = threadIdx.x; c < C; c += NW * 64) {
            float tot = s_dw[c];
#pragma unroll
            for (int r = 1; r < NR; ++r) tot += s_dw[r * C + c];
            if (h.nleaf == 1)
                store_dyn(dw_row, h.w_dtype, c, tot);
            else
                mine[c] = tot;
        }
    }
}

// Rows beyond the register-resident limit: a workgroup of 256 lanes owns one row at a time and streams over it
// twice, lane t handling the chunks t, t+256, t+512, ... of VEC elements: the first pass accumulates the
// row statistics, the second re-reads x (and dy, w) -- the row was just read, so this comes from L2 -- and
// writes the result.  Only the dw sums of the RMSNorm backward stay in registers (NKW chunks per lane, a
// compile-time bound; 0 when there is no dw); since every channel belongs to exactly one lane of the
// workgroup, the block's partial dw row is written straight from them.  Rows with more than NKW chunks per
// lane are covered by gridDim.z channel slabs of 256 * NKW * VEC channels: the blocks of slab 0 do everything
// above and keep the dw sums of the first slab, the blocks of slab z > 0 recompute the row statistic from x and
// keep the dw sums of their own slab only (they write no dx), so any width works and every sum keeps its
// fixed order.
template <typename T, int OP, bool BWD, int VEC, bool VECTOR, int NKW>
__global__ __launch_bounds__(256) void wide_stream_kernel(const WideParams p) {
    __shared__ float s_red[2][2][4];  // [parity][statistic][wavefront]
    constexpr bool HAS_W = (OP == WIDE_RMS);
    const int which = (int)blockIdx.x >= p.h[0].nchunks ? 1 : 0;
    const WideHalf& h = p.h[which];
    const int chunk = blockIdx.x - (which ? p.h[0].nchunks : 0);
    const int b = blockIdx.y;
    const int C = h.C;
    const int r0 = chunk * p.rows_per_chunk;
    const int r1 = min(h.T, r0 + p.rows_per_chunk);
    const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
    const int nk = (C + 256 * VEC - 1) / (256 * VEC);  // chunks per lane
    const int k0 = NKW > 0 ? (int)blockIdx.z * NKW : 0;  // first chunk of this block's dw slab
    const bool lead = blockIdx.z == 0;                    // this block also produces dx
    if (k0 >= nk) return;  // the narrower of two tensors may have fewer slabs (block-uniform)

    const T* xb = static_cast<const T*>(h.x) + (int64_t)b * h.sx_b;
    const T* db = BWD ? static_cast<const T*>(h.dy) + (int64_t)b * h.sd_b : nullptr;
    T* yb = static_cast<T*>(h.y) + (int64_t)b * h.sy_b;
    const char* wp = HAS_W ? static_cast<const char*>(h.w) + (int64_t)b * h.sw_b * (h.w_dtype == RGD_F32 ? 4 : 2) : nullptr;
    const bool w_vec = VECTOR && h.w_vec;
    auto load_w = [&](int first, float (&w)[VEC]) {
        if (w_vec)
            load_chunk_dyn<VEC, VECTOR>(wp, h.w_dtype, first, C, w);
        else
            load_chunk_dyn<VEC, false>(wp, h.w_dtype, first, C, w);
    };

    constexpr int NACC = NKW > 0 ? NKW : 1;
    float dwacc[NACC][VEC];
#pragma unroll
    for (int k = 0; k < NACC; ++k)
#pragma unroll
        for (int e = 0; e < VEC; ++e) dwacc[k][e] = 0.f;

    for (int r = r0; r < r1; ++r) {
        const T* xr = xb + (int64_t)r * h.sx_n;
        const T* dr = BWD ? db + (int64_t)r * h.sd_n : nullptr;
        // ---- pass 1: sum x^2 (and sum x*dy*w) ----
        float ss = 0.f, sd = 0.f;
        for (int k = 0; k < nk; ++k) {
            const int first = (k * 256 + tid) * VEC;
            float xv[VEC], dv[VEC], wv[VEC];
            load_chunk<T, VEC, VECTOR>(xr, first, C, xv);
            if constexpr (BWD) {
                if (lead) {
                    load_chunk<T, VEC, VECTOR>(dr, first, C, dv);
                    if constexpr (HAS_W) load_w(first, wv);
                }
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                ss += xv[e] * xv[e];
                if constexpr (BWD) {
                    if (lead) sd += xv[e] * (HAS_W ? dv[e] * wv[e] : dv[e]);
                }
            }
        }
        ss = group_reduce<64>(ss);
        if constexpr (BWD) sd = group_reduce<64>(sd);
        const int par = (r - r0) & 1;
        if (lane == 0) {
            s_red[par][0][wave] = ss;
            if constexpr (BWD) s_red[par][1][wave] = sd;
        }
        __syncthreads();
        ss = (s_red[par][0][0] + s_red[par][0][1]) + (s_red[par][0][2] + s_red[par][0][3]);
        if constexpr (BWD) sd = (s_red[par][1][0] + s_red[par][1][1]) + (s_red[par][1][2] + s_red[par][1][3]);
        float rn;  // rrms or rlen
        if constexpr (OP == WIDE_RMS) {
            rn = rsqrtf(ss * h.inv_c + p.eps);
        } else {
            const float len = sqrtf(ss);
            rn = len < p.eps ? 1.0f / p.eps : 1.0f / len;
        }
        const float inner = OP == WIDE_RMS ? sd * rn * h.inv_c : sd * rn;
        // ---- pass 2: results ----
        T* yr = yb + (int64_t)r * h.sy_n;
        auto body = [&](int k, float (&acc)[VEC]) {
            const int first = (k * 256 + tid) * VEC;
            float xv[VEC], dv[VEC], wv[VEC], out[VEC];
            load_chunk<T, VEC, VECTOR>(xr, first, C, xv);
            if constexpr (BWD) load_chunk<T, VEC, VECTOR>(dr, first, C, dv);
            if constexpr (HAS_W) load_w(first, wv);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (!BWD) {
                    out[e] = HAS_W ? xv[e] * rn * wv[e] : xv[e] * rn;
                } else {
                    const float xh = xv[e] * rn;
                    const float gr = HAS_W ? dv[e] * wv[e] : dv[e];
                    out[e] = (gr - xh * inner) * rn;
                    if constexpr (NKW > 0) acc[e] += xh * dv[e];
                }
            }
            store_chunk<T, VEC, VECTOR>(yr, first, C, out);
        };
        if constexpr (NKW > 0) {
            if (lead) {
#pragma unroll
                for (int k = 0; k < NKW; ++k)
                    if (k < nk) body(k, dwacc[k]);
                float unused[VEC] = {};
                for (int k = NKW; k < nk; ++k) body(k, unused);  // chunks whose dw sums belong to later slabs
            } else {
                // dw sums of this slab only: xhat * dy
#pragma unroll
                for (int k = 0; k < NKW; ++k) {
                    if (k0 + k < nk) {
                        const int first = ((k0 + k) * 256 + tid) * VEC;
                        float xv[VEC], dv[VEC];
                        load_chunk<T, VEC, VECTOR>(xr, first, C, xv);
                        load_chunk<T, VEC, VECTOR>(dr, first, C, dv);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) dwacc[k][e] += xv[e] * rn * dv[e];
                    }
                }
            }
        } else {
            for (int k = 0; k < nk; ++k) body(k, dwacc[0]);
        }
    }

    if constexpr (NKW > 0) {
        const int wgt = h.w_shared ? 0 : b;
        const int idx = h.w_shared ? b * h.nchunks + chunk : chunk;
        void* dw_row = static_cast<char*>(h.dw) + (int64_t)wgt * h.sdw_b * (h.w_dtype == RGD_F32 ? 4 : 2);
        float* mine = h.part + ((int64_t)wgt * h.nleaf + idx) * C;
#pragma unroll
        for (int k = 0; k < NKW; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int c = ((k0 + k) * 256 + tid) * VEC + e;
                if (c < C) {
                    if (h.nleaf == 1)
                        store_dyn(dw_row, h.w_dtype, c, dwacc[k][e]);
                    else
                        mine[c] = dwacc[k][e];
                }
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
                int dtype, float eps, void* workspace, size_t workspace_bytes, void* stream);
size_t wide_workspace(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2);
// bytes of the library-owned scratch array behind rgd_rms_bwd_noalloc (one copy per GPU, held for the process' life)
#ifndef RGD_NOALLOC_SCRATCH_BYTES
#define RGD_NOALLOC_SCRATCH_BYTES (16u << 20)
#endif
int wide_noalloc_setup(void** out);  // rows_wide.hip: address of that array on the current device

// per-dtype instantiation units (rows_wide_f32.hip, rows_wide_f16.hip, rows_wide_bf16.hip)
struct WideConfig {
    int op;
    bool bwd;
    int G, NV, WPR;
    bool vector;
    bool stream;  // rows beyond the register-resident limit: wide_stream_kernel
};
// chunks of dw sums a lane of the streaming RMSNorm backward holds: at most 64 fp32 accumulators
constexpr int wide_stream_nkw(int vec) { return vec >= 4 ? 64 / vec : 16; }
// compile-time launch shape shared by the kernel instantiations and the host-side grid computation
// rows a lane group has in flight at once, by the elements of one row a lane holds (nv chunks of vec)
constexpr int wide_unroll(bool bwd, int nv, int vec) {
    return bwd ? (nv * vec <= RGD_WIDE_EPL_U2 ? 2 : 1) : (nv * vec <= 8 ? 4 : (nv * vec <= 16 ? 2 : 1));
}
constexpr int wide_waves(int op, bool bwd) { return (bwd && op == WIDE_RMS) ? 8 : 4; }
template <typename T> int wide_dispatch(const WideConfig& cfg, const WideParams& p, dim3 grid, size_t lds, hipStream_t s);
