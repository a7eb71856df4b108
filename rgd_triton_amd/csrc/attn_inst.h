// Instantiates the attention kernels for one element type and dispatches run-time head dim / bias kind.
// Included by attn_f16.hip and attn_bf16.hip.
#pragma once

#include "attn_fwd.h"
#include "attn_bwd.h"

template <typename T, int DPAD, int BIAS> int launch_fwd(const AttnFwdParams& p, unsigned grid, hipStream_t s) {
    auto kern = attn_fwd_kernel<T, DPAD, BIAS>;
    constexpr size_t lds = AttnFwdSmem<DPAD>::BYTES;
    static bool configured = false;  // benign race: the attribute is idempotent
    if (!configured && lds > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess) {
            rgd_set_error("rgd_attn_fwd: cannot reserve %zu bytes of LDS", lds);
            return RGD_ERR_LAUNCH;
        }
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(ATTN_THREADS), lds, s, p);
    return RGD_OK;
}

template <typename T, int DPAD> int launch_fwd_merge(const AttnFwdParams& p, unsigned items, hipStream_t s) {
    const unsigned gy = (ATTN_BM * (DPAD / 4) + 255) / 256;
    hipLaunchKernelGGL((attn_fwd_merge_kernel<T, DPAD>), dim3(items, gy), dim3(256), 0, s, p);
    return RGD_OK;
}

template <typename T> int dispatch_fwd_merge(const AttnFwdParams& p, unsigned items, hipStream_t s) {
    if (p.D <= 32) return launch_fwd_merge<T, 32>(p, items, s);
    if (p.D <= 64) return launch_fwd_merge<T, 64>(p, items, s);
    if (p.D <= 96) return launch_fwd_merge<T, 96>(p, items, s);
    return launch_fwd_merge<T, 128>(p, items, s);
}

template <typename T> int dispatch_fwd(const AttnFwdParams& p, unsigned grid, hipStream_t s) {
    const int bias = p.bias_kind == RGD_BIAS_NONE ? BIAS_OFF : (p.bias_dtype == RGD_F32 ? BIAS_F32 : BIAS_SAME);
#define FWD_CASE(DP)                                                                 \
    if (p.D <= DP)                                                                   \
        return bias == BIAS_OFF    ? launch_fwd<T, DP, BIAS_OFF>(p, grid, s)         \
               : bias == BIAS_SAME ? launch_fwd<T, DP, BIAS_SAME>(p, grid, s)        \
                                   : launch_fwd<T, DP, BIAS_F32>(p, grid, s);
    FWD_CASE(32)
    FWD_CASE(64)
    FWD_CASE(96)
    FWD_CASE(128)
#undef FWD_CASE
    return RGD_ERR_UNSUPPORTED;
}

template <typename T, int DPAD, int BIAS, bool DQ> int launch_bwd(const AttnBwdParams& p, unsigned grid, hipStream_t s) {
    auto kern = DQ ? attn_bwd_dq_kernel<T, DPAD, BIAS> : attn_bwd_dkv_kernel<T, DPAD, BIAS>;
    constexpr size_t lds = DQ ? DqSmem<DPAD>::BYTES : DkvSmem<DPAD, dkv_nsub(DPAD, BIAS)>::BYTES;
    static bool configured = false;
    if (!configured && lds > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess) {
            rgd_set_error("rgd_attn_bwd: cannot reserve %zu bytes of LDS", lds);
            return RGD_ERR_LAUNCH;
        }
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(BWD_THREADS), lds, s, p);
    return RGD_OK;
}

template <typename T, bool DQ> int dispatch_bwd(const AttnBwdParams& p, unsigned grid, hipStream_t s) {
    const int bias = p.bias_kind == RGD_BIAS_NONE ? BIAS_OFF : (p.bias_dtype == RGD_F32 ? BIAS_F32 : BIAS_SAME);
#define BWD_CASE(DP)                                                                     \
    if (p.D <= DP)                                                                       \
        return bias == BIAS_OFF    ? launch_bwd<T, DP, BIAS_OFF, DQ>(p, grid, s)         \
               : bias == BIAS_SAME ? launch_bwd<T, DP, BIAS_SAME, DQ>(p, grid, s)        \
                                   : launch_bwd<T, DP, BIAS_F32, DQ>(p, grid, s);
    BWD_CASE(32)
    BWD_CASE(64)
    BWD_CASE(96)
    BWD_CASE(128)
#undef BWD_CASE
    return RGD_ERR_UNSUPPORTED;
}


template <typename T, int DPAD> int launch_bwd_merge(const AttnBwdParams& p, unsigned items, int nt, hipStream_t s) {
    const unsigned gy = (BWD_BM * (DPAD / 4) + 255) / 256;
    hipLaunchKernelGGL((attn_bwd_merge_kernel<T, DPAD>), dim3(items, gy, nt), dim3(256), 0, s, p, nt);
    return RGD_OK;
}

template <typename T> int dispatch_bwd_merge(const AttnBwdParams& p, unsigned items, int nt, hipStream_t s) {
    if (p.D <= 32) return launch_bwd_merge<T, 32>(p, items, nt, s);
    if (p.D <= 64) return launch_bwd_merge<T, 64>(p, items, nt, s);
    if (p.D <= 96) return launch_bwd_merge<T, 96>(p, items, nt, s);
    return launch_bwd_merge<T, 128>(p, items, nt, s);
}
