// Host side of the (B,T,C) row kernels: argument validation, configuration choice, workspace layout
// and the extern "C" entry points for RMSNorm / RMSNorm2 / L2 / L2x2.
#include "rows_wide.h"

#include <algorithm>
#include <atomic>
#include <mutex>
#include <string.h>

#ifndef RGD_DW_BLOCKS_PER_CU
#define RGD_DW_BLOCKS_PER_CU 1
#endif

namespace {

constexpr int DW_BLOCKS_PER_CU = RGD_DW_BLOCKS_PER_CU;  // blocks (= partial dw rows) per compute unit, RMSNorm backward
constexpr int BLOCKS_PER_CU = 8;     // target grid size of the other kernels

int pow2ceil(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

// upper bound of the partial rows one half can need, whatever tile shape is chosen later
size_t half_bound(int64_t B, int64_t T, int64_t target) {
    return T <= 0 ? 0 : (size_t)target + (size_t)B + 8;
}

// dw[weight][c] = sum over the partial rows of that weight, in a fixed order: wavefront w of the block adds
// rows w, w+WAVES, w+2*WAVES, ... for 64 consecutive channels, then the wavefront sums are added in index order.
__global__ __launch_bounds__(WIDE_RED_WAVES * 64) void wide_dw_reduce_kernel(const WideParams p) {
    __shared__ float s_sum[WIDE_RED_WAVES][64];
    const int which = (int)blockIdx.x >= p.h[0].red_blocks ? 1 : 0;
    const WideHalf& h = p.h[which];
    const int blk = blockIdx.x - (which ? p.h[0].red_blocks : 0);
    const int cblocks = (h.C + 63) / 64;
    const int wgt = blk / cblocks;
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    const int c = (blk - wgt * cblocks) * 64 + lane;
    const float* src = h.part + (int64_t)wgt * h.nleaf * h.C + c;
    float acc = 0.f;
    if (c < h.C) {
        int r = wave;
        // the partial rows were written by other compute units moments ago, so every read is a trip to the
        // memory side: eight independent reads in flight per lane, added in row order
#pragma unroll 1
        for (; r + 7 * WIDE_RED_WAVES < h.nleaf; r += 8 * WIDE_RED_WAVES) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = src[(int64_t)(r + i * WIDE_RED_WAVES) * h.C];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc += v[i];
        }
        for (; r < h.nleaf; r += WIDE_RED_WAVES) acc += src[(int64_t)r * h.C];
    }
    s_sum[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && c < h.C) {
        float tot = s_sum[0][lane];
#pragma unroll
        for (int w = 1; w < WIDE_RED_WAVES; ++w) tot += s_sum[w][lane];
        void* dw_row = static_cast<char*>(h.dw) + (int64_t)wgt * h.sdw_b * (h.w_dtype == RGD_F32 ? 4 : 2);
        store_dyn(dw_row, h.w_dtype, c, tot);
    }
}

bool t3_vec_ok(const rgd_tensor3* t, int es) {
    return t && rgd_aligned16(t->ptr) && (t->stride_b * es) % 16 == 0 && (t->stride_n * es) % 16 == 0;
}

}  // namespace

size_t wide_workspace(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2) {
    const int64_t target = (int64_t)rgd_num_cus() * DW_BLOCKS_PER_CU;
    const size_t r1 = half_bound(B, T1, target), r2 = half_bound(B, T2, target);
    return (r1 * (size_t)std::max<int64_t>(C1, 0) + r2 * (size_t)std::max<int64_t>(C2, 0)) * sizeof(float);
}

int wide_launch(const char* name, int op, bool bwd, int64_t B, const WideHalfArgs& a1, const WideHalfArgs& a2,
                int dtype, float eps, void* workspace, size_t workspace_bytes, void* stream) {
    rgd_ensure_init();
    RGD_REQUIRE(rgd_dtype_ok(dtype), RGD_ERR_INVALID, "%s: Only support fp16, bf16, and fp32", name);
    RGD_REQUIRE(B >= 0 && B <= 65535, RGD_ERR_INVALID, "%s: batch %lld out of range", name, (long long)B);
    const WideHalfArgs* as[2] = {&a1, &a2};
    const int es = rgd_dtype_size(dtype);
    const bool has_w = op == WIDE_RMS;
    bool vector = true;
    int64_t maxC = 0, total_rows = 0;
    for (const WideHalfArgs* a : as) {
        RGD_REQUIRE(a->T >= 0 && a->T < (1ll << 31) && a->C >= 0 && a->C < (1ll << 31), RGD_ERR_INVALID,
                    "%s: shape out of range", name);
        if (B == 0 || a->T == 0 || a->C == 0) continue;  // nothing to do for this tensor (its pointers may be null)
        RGD_REQUIRE(a->x && a->x->ptr && a->y && a->y->ptr, RGD_ERR_INVALID, "%s: null tensor", name);
        RGD_REQUIRE(!bwd || (a->dy && a->dy->ptr), RGD_ERR_INVALID, "%s: null gradient", name);
        RGD_REQUIRE(!has_w || (a->w && a->w->ptr && rgd_dtype_ok(a->w_dtype)), RGD_ERR_INVALID, "%s: bad weight", name);
        RGD_REQUIRE(!(has_w && bwd) || (a->dw && a->dw->ptr), RGD_ERR_INVALID, "%s: null dw", name);
        vector = vector && (a->C * es) % 16 == 0 && t3_vec_ok(a->x, es) && t3_vec_ok(a->y, es) &&
                 (!bwd || t3_vec_ok(a->dy, es));
        maxC = std::max(maxC, a->C);
        total_rows += B * a->T;
    }
    if (total_rows == 0 || B == 0) return RGD_OK;

    WideConfig cfg;
    cfg.op = op;
    cfg.bwd = bwd;
    cfg.vector = vector;
    const int vec = vector ? 16 / es : 2;
    const int64_t chunks = (maxC + vec - 1) / vec;
    // elements of one row a lane may hold: x (+ dy) (+ w and the dw accumulators) all stay in registers; the
    // RMSNorm forward keeps only x and reads w as it goes, so it takes the wider limit (one wavefront per row up to
    // 4096 channels instead of four: no barrier per row, 6 % faster at C = 4096)
    const int max_epl = (has_w && (bwd || !RGD_WIDE_RMS_FWD_64)) ? 32 : 64;
    cfg.WPR = 1;
    cfg.NV = 0;
    if (chunks <= 64) {
        cfg.G = std::max(4, pow2ceil((int)chunks));
        cfg.NV = 1;
    } else {
        cfg.G = 64;
        static const int allowed1[] = {2, 3, 4, 6, 8, 12, 16};
        static const int allowed4[] = {1, 2, 3, 4, 6, 8, 12, 16};
        const int64_t need1 = (chunks + 63) / 64, need4 = (chunks + 255) / 256;
        for (int nv : allowed1)
            if (nv >= need1 && nv * vec <= max_epl) {
                cfg.NV = nv;
                break;
            }
        if (cfg.NV == 0) {  // too wide for one wavefront: four wavefronts share a row
            cfg.WPR = 4;
            for (int nv : allowed4)
                if (nv >= need4 && nv * vec <= max_epl) {
                    cfg.NV = nv;
                    break;
                }
        }
    }
    cfg.stream = cfg.NV == 0;  // too wide for registers: the two-pass streaming kernel
    int64_t slabs = 1;  // channel slabs of the streaming RMSNorm backward (its dw sums stay in registers, slab by slab)
    if (cfg.stream) {
        if (has_w && bwd) {
            const int64_t slab_channels = (int64_t)256 * wide_stream_nkw(vec) * vec;
            slabs = (maxC + slab_channels - 1) / slab_channels;
            RGD_REQUIRE(slabs <= 65535, RGD_ERR_UNSUPPORTED, "%s: rows of %lld elements are too wide", name, (long long)maxC);
        }
        cfg.G = 64;
        cfg.NV = 1;
        cfg.WPR = 4;
    }
    const int NW = cfg.stream ? 4 : wide_waves(op, bwd);
    const int U = cfg.stream ? 1 : wide_unroll(bwd, cfg.NV, vec);
    const int row_quantum = cfg.stream ? 1 : NW * (64 / cfg.G) / cfg.WPR * U;
    const bool tree = has_w && bwd;
    const int64_t target = (int64_t)rgd_num_cus() * (tree ? DW_BLOCKS_PER_CU : BLOCKS_PER_CU);
    int64_t rpc = (total_rows + target - 1) / target;
    rpc = std::max<int64_t>(row_quantum, (rpc + row_quantum - 1) / row_quantum * row_quantum);
    RGD_REQUIRE(rpc < (1ll << 30), RGD_ERR_UNSUPPORTED, "%s: too many rows", name);

    WideParams p;
    memset(&p, 0, sizeof(p));
    p.rows_per_chunk = (int)rpc;
    p.eps = eps;
    size_t ws_used = 0;
    int64_t grid_x = 0, red_grid = 0;
    for (int i = 0; i < 2; ++i) {
        const WideHalfArgs* a = as[i];
        WideHalf& h = p.h[i];
        if (a->T == 0 || a->C == 0) {
            h.nchunks = 0;
            continue;
        }
        h.x = a->x->ptr;
        h.sx_b = a->x->stride_b;
        h.sx_n = a->x->stride_n;
        h.y = a->y->ptr;
        h.sy_b = a->y->stride_b;
        h.sy_n = a->y->stride_n;
        if (bwd) {
            h.dy = a->dy->ptr;
            h.sd_b = a->dy->stride_b;
            h.sd_n = a->dy->stride_n;
        }
        h.T = (int)a->T;
        h.C = (int)a->C;
        h.inv_c = 1.0f / (float)a->C;
        h.nchunks = (int)((a->T + rpc - 1) / rpc);
        grid_x += h.nchunks;
        if (has_w) {
            const int ws_ = rgd_dtype_size(a->w_dtype);
            h.w = a->w->ptr;
            h.sw_b = a->w->stride_b;
            h.w_dtype = a->w_dtype;
            h.w_vec = rgd_aligned16(a->w->ptr) && (a->w->stride_b * ws_) % 16 == 0 && (a->C * ws_) % 16 == 0 &&
                      (vec * ws_) % 16 == 0;
        }
        if (tree) {
            h.dw = a->dw->ptr;
            h.sdw_b = a->dw->stride_b;
            h.w_shared = a->w_shared ? 1 : 0;
            h.nleaf = h.w_shared ? (int)B * h.nchunks : h.nchunks;
            const int nweights = h.w_shared ? 1 : (int)B;
            h.part = reinterpret_cast<float*>(static_cast<char*>(workspace) + ws_used);
            if (h.nleaf > 1) {
                ws_used += (size_t)nweights * h.nleaf * a->C * sizeof(float);
                h.red_blocks = nweights * (int)((a->C + 63) / 64);
                red_grid += h.red_blocks;
            }
        }
    }
    if (tree) {
        RGD_REQUIRE(ws_used <= workspace_bytes, RGD_ERR_WORKSPACE, "%s: workspace too small (need %zu bytes, have %zu)",
                    name, ws_used, workspace_bytes);
        RGD_REQUIRE(ws_used == 0 || workspace, RGD_ERR_INVALID, "%s: null workspace", name);
    }
    RGD_REQUIRE(grid_x < (1ll << 31), RGD_ERR_UNSUPPORTED, "%s: grid too large", name);

    const dim3 grid((unsigned)grid_x, (unsigned)B, (unsigned)slabs);
    // one row of dw sums per wavefront group (the streaming kernel writes its sums from registers)
    const size_t lds = (tree && !cfg.stream) ? (size_t)(NW / cfg.WPR) * maxC * sizeof(float) : 0;
    RGD_REQUIRE(lds <= 64 * 1024, RGD_ERR_UNSUPPORTED, "%s: row too wide for the dw staging buffer", name);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc;
    if (dtype == RGD_F32)
        rc = wide_dispatch<float>(cfg, p, grid, lds, s);
    else if (dtype == RGD_F16)
        rc = wide_dispatch<f16_t>(cfg, p, grid, lds, s);
    else
        rc = wide_dispatch<bf16_t>(cfg, p, grid, lds, s);
    if (rc != RGD_OK) return rc;
    if (red_grid > 0)  // dw = fixed-order sum of the blocks' partial rows
        return rgd_launch_status(name, rgd_launch(wide_dw_reduce_kernel, dim3((unsigned)red_grid), dim3(WIDE_RED_WAVES * 64), 0, s, p));
    return RGD_OK;
}

// ------------------------------------------------------------------------------------------
// Scratch owned by the library, for the entry point that must not allocate (rgd_rms_bwd_noalloc): the partial dw
// rows live in this file-scope device array instead of a caller's workspace.  Every GPU the library runs on holds
// its own copy of the array, at its own address, until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress; the address that call returns for a device is what kernels and runtime calls get.
// ------------------------------------------------------------------------------------------
constexpr size_t kNoAllocScratchBytes = RGD_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;
}  // namespace

// Resolves the scratch array's address on the CURRENT device (once per device); *out receives it.
int wide_noalloc_setup(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        rgd_set_error("rgd_rms_bwd_noalloc: no current device (or a device index of %d or more)", kMaxDevices);
        return RGD_ERR_INVALID;
    }
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!ptr) {
            const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !ptr) {
                (void)hipGetLastError();
                rgd_set_error("rgd_rms_bwd_noalloc: hipGetSymbolAddress(scratch) failed on device %d: %s", dev,
                              hipGetErrorString(e));
                return RGD_ERR_LAUNCH;
            }
            g_scratch_ptr[dev].store(ptr, std::memory_order_release);
        }
    }
    if (out) *out = ptr;
    return RGD_OK;
}

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------
namespace {
WideHalfArgs half(int64_t T, int64_t C, const rgd_tensor3* x, const rgd_tensor3* dy, const rgd_tensor3* y,
                  const rgd_tensor3* w = nullptr, const rgd_tensor3* dw = nullptr, int w_dtype = RGD_F32,
                  int w_shared = 0) {
    WideHalfArgs a;
    a.T = T;
    a.C = C;
    a.x = x;
    a.dy = dy;
    a.y = y;
    a.w = w;
    a.dw = dw;
    a.w_dtype = w_dtype;
    a.w_shared = w_shared;
    return a;
}
const WideHalfArgs kNoHalf;
}  // namespace

extern "C" {

int rgd_rms_fwd(int64_t B, int64_t T, int64_t C, const rgd_tensor3* x, const rgd_tensor3* w, const rgd_tensor3* y,
                int x_dtype, int w_dtype, float eps, void* stream) {
    return wide_launch("rgd_rms_fwd", WIDE_RMS, false, B, half(T, C, x, nullptr, y, w, nullptr, w_dtype), kNoHalf,
                       x_dtype, eps, nullptr, 0, stream);
}

size_t rgd_rms_bwd_workspace(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2) {
    return wide_workspace(B, T1, C1, T2, C2);
}

int rgd_rms_bwd(int64_t B, int64_t T, int64_t C, const rgd_tensor3* dy, const rgd_tensor3* x, const rgd_tensor3* w,
                const rgd_tensor3* dx, const rgd_tensor3* dw, int w_shared, int x_dtype, int w_dtype, float eps,
                void* workspace, size_t workspace_bytes, void* stream) {
    return wide_launch("rgd_rms_bwd", WIDE_RMS, true, B, half(T, C, x, dy, dx, w, dw, w_dtype, w_shared), kNoHalf,
                       x_dtype, eps, workspace, workspace_bytes, stream);
}

size_t rgd_rms_bwd_noalloc_limit(void) { return kNoAllocScratchBytes; }

int rgd_rms_bwd_noalloc(int64_t B, int64_t T, int64_t C, const rgd_tensor3* dy, const rgd_tensor3* x,
                        const rgd_tensor3* w, const rgd_tensor3* dx, const rgd_tensor3* dw, int w_shared, int x_dtype,
                        int w_dtype, float eps, void* stream) {
    const char* name = "rgd_rms_bwd_noalloc";
    rgd_ensure_init();
    // the size rgd_rms_bwd_workspace asks a caller for must fit the fixed array
    RGD_REQUIRE(B >= 0 && T >= 0 && C >= 0, RGD_ERR_INVALID, "%s: negative shape", name);
    const size_t need = wide_workspace(B, T, C, 0, 0);
    RGD_REQUIRE(need <= kNoAllocScratchBytes, RGD_ERR_WORKSPACE,
                "%s: (B=%lld, T=%lld, C=%lld) needs %zu bytes of scratch, the library's fixed scratch holds %zu; use "
                "rgd_rms_bwd with a workspace", name, (long long)B, (long long)T, (long long)C, need,
                kNoAllocScratchBytes);
    void* ptr = nullptr;
    const int rc = wide_noalloc_setup(&ptr);  // hipGetDevice and one atomic load once the device has been seen
    if (rc != RGD_OK) return rc;
    // every partial row the reduce kernel reads is written by this call's first kernel: nothing has to start at 0
    return wide_launch(name, WIDE_RMS, true, B, half(T, C, x, dy, dx, w, dw, w_dtype, w_shared), kNoHalf, x_dtype, eps,
                       ptr, kNoAllocScratchBytes, stream);
}

int rgd_fused_rms_fwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2, const rgd_tensor3* x1,
                      const rgd_tensor3* w1, const rgd_tensor3* y1, const rgd_tensor3* x2, const rgd_tensor3* w2,
                      const rgd_tensor3* y2, int x_dtype, int w1_dtype, int w2_dtype, float eps, void* stream) {
    return wide_launch("rgd_fused_rms_fwd", WIDE_RMS, false, B, half(T1, C1, x1, nullptr, y1, w1, nullptr, w1_dtype),
                       half(T2, C2, x2, nullptr, y2, w2, nullptr, w2_dtype), x_dtype, eps, nullptr, 0, stream);
}

int rgd_fused_rms_bwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2, const rgd_tensor3* dy1,
                      const rgd_tensor3* x1, const rgd_tensor3* w1, const rgd_tensor3* dx1, const rgd_tensor3* dw1,
                      int w1_shared, const rgd_tensor3* dy2, const rgd_tensor3* x2, const rgd_tensor3* w2,
                      const rgd_tensor3* dx2, const rgd_tensor3* dw2, int w2_shared, int x_dtype, int w1_dtype,
                      int w2_dtype, float eps, void* workspace, size_t workspace_bytes, void* stream) {
    return wide_launch("rgd_fused_rms_bwd", WIDE_RMS, true, B, half(T1, C1, x1, dy1, dx1, w1, dw1, w1_dtype, w1_shared),
                       half(T2, C2, x2, dy2, dx2, w2, dw2, w2_dtype, w2_shared), x_dtype, eps, workspace,
                       workspace_bytes, stream);
}

int rgd_l2_fwd(int64_t B, int64_t T, int64_t C, const rgd_tensor3* x, const rgd_tensor3* y, int dtype, float eps,
               void* stream) {
    return wide_launch("rgd_l2_fwd", WIDE_L2, false, B, half(T, C, x, nullptr, y), kNoHalf, dtype, eps, nullptr, 0, stream);
}

int rgd_l2_bwd(int64_t B, int64_t T, int64_t C, const rgd_tensor3* dy, const rgd_tensor3* x, const rgd_tensor3* dx,
               int dtype, float eps, void* stream) {
    return wide_launch("rgd_l2_bwd", WIDE_L2, true, B, half(T, C, x, dy, dx), kNoHalf, dtype, eps, nullptr, 0, stream);
}

int rgd_fused_l2_fwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2, const rgd_tensor3* x1,
                     const rgd_tensor3* y1, const rgd_tensor3* x2, const rgd_tensor3* y2, int dtype, float eps,
                     void* stream) {
    return wide_launch("rgd_fused_l2_fwd", WIDE_L2, false, B, half(T1, C1, x1, nullptr, y1),
                       half(T2, C2, x2, nullptr, y2), dtype, eps, nullptr, 0, stream);
}

int rgd_fused_l2_bwd(int64_t B, int64_t T1, int64_t C1, int64_t T2, int64_t C2, const rgd_tensor3* dy1,
                     const rgd_tensor3* x1, const rgd_tensor3* dx1, const rgd_tensor3* dy2, const rgd_tensor3* x2,
                     const rgd_tensor3* dx2, int dtype, float eps, void* stream) {
    return wide_launch("rgd_fused_l2_bwd", WIDE_L2, true, B, half(T1, C1, x1, dy1, dx1), half(T2, C2, x2, dy2, dx2),
                       dtype, eps, nullptr, 0, stream);
}

}  // extern "C"
