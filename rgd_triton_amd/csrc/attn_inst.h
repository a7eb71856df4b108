// Instantiates the attention kernels for one element type and dispatches run-time head dim / bias kind.
// Included by attn_f16.hip and attn_bf16.hip.
#pragma once

#include "attn_fwd.h"
#include "attn_bwd.h"

template <typename T, int DPAD, int BIAS> int launch_fwd(const AttnFwdParams& p, unsigned grid, hipStream_t s) {
    constexpr size_t lds = AttnFwdSmem<DPAD>::BYTES;  // its attribute was set by attn_configure_all
    return rgd_launch_status("rgd_attn_fwd", rgd_launch(attn_fwd_kernel<T, DPAD, BIAS>, dim3(grid), dim3(ATTN_THREADS), lds, s, p));
}

template <typename T, int DPAD> int launch_fwd_merge(const AttnFwdParams& p, unsigned items, hipStream_t s) {
    const unsigned gy = (ATTN_BM * (DPAD / 4) + 255) / 256;
    return rgd_launch_status("rgd_attn_fwd (merge)", rgd_launch(attn_fwd_merge_kernel<T, DPAD>, dim3(items, gy), dim3(256), 0, s, p));
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
    constexpr size_t lds = DQ ? DqSmem<DPAD>::BYTES : DkvSmem<DPAD, dkv_nsub(DPAD, BIAS)>::BYTES;
    if constexpr (DQ && BIAS != BIAS_OFF) {
        if (p.dbias.ptr)  // the variant that also writes the bias gradient
            return rgd_launch_status("rgd_attn_bwd", rgd_launch(attn_bwd_dq_kernel<T, DPAD, BIAS, true>, dim3(grid),
                                                                dim3(BWD_THREADS), lds, s, p));
    }
    auto kern = DQ ? attn_bwd_dq_kernel<T, DPAD, BIAS> : attn_bwd_dkv_kernel<T, DPAD, BIAS>;
    return rgd_launch_status("rgd_attn_bwd", rgd_launch(kern, dim3(grid), dim3(BWD_THREADS), lds, s, p));
}

// ---- one-pass backward (head dims up to 64): prep -> fused key-block kernel -> dQ convert ----
template <typename T, int DPAD, int BIAS> int launch_bwd_fused(const AttnBwdParams& p, unsigned grid, hipStream_t s) {
    constexpr size_t lds = DkvSmem<DPAD, dkv_nsub(DPAD, BIAS, true), true>::BYTES;
    return rgd_launch_status("rgd_attn_bwd (one pass)",
                             rgd_launch(attn_bwd_dkv_kernel<T, DPAD, BIAS, true>, dim3(grid), dim3(BWD_THREADS), lds, s, p));
}
template <typename T> int dispatch_bwd_fused(const AttnBwdParams& p, unsigned grid, hipStream_t s) {
    const int bias = p.bias_kind == RGD_BIAS_NONE ? BIAS_OFF : (p.bias_dtype == RGD_F32 ? BIAS_F32 : BIAS_SAME);
#define FUSED_CASE(DP)                                                                 \
    if (p.D <= DP)                                                                     \
        return bias == BIAS_OFF    ? launch_bwd_fused<T, DP, BIAS_OFF>(p, grid, s)     \
               : bias == BIAS_SAME ? launch_bwd_fused<T, DP, BIAS_SAME>(p, grid, s)    \
                                   : launch_bwd_fused<T, DP, BIAS_F32>(p, grid, s);
    FUSED_CASE(32)
    FUSED_CASE(64)
#undef FUSED_CASE
    rgd_set_error("rgd_attn_bwd: the one-pass form covers head dims up to 64");
    return RGD_ERR_UNSUPPORTED;
}
// which = 0: delta and a cleared dq_accum before the main kernel; 1: dq from dq_accum after it
template <typename T> int dispatch_bwd_fused_aux(const AttnBwdParams& p, int which, hipStream_t s) {
    const int dpad = p.D <= 32 ? 32 : 64;
    const int rows_per_block = 256 / (dpad / 8);
    const int64_t rows = (int64_t)p.B * p.H * (which == 0 ? p.Tq_rounded : p.Tq);
    const dim3 grid((unsigned)((rows + rows_per_block - 1) / rows_per_block));
    hipError_t e;
    if (which == 0)
        e = dpad == 32 ? rgd_launch(attn_bwd_prep_kernel<T, 32>, grid, dim3(256), 0, s, p)
                       : rgd_launch(attn_bwd_prep_kernel<T, 64>, grid, dim3(256), 0, s, p);
    else
        e = dpad == 32 ? rgd_launch(attn_bwd_dq_convert_kernel<T, 32>, grid, dim3(256), 0, s, p)
                       : rgd_launch(attn_bwd_dq_convert_kernel<T, 64>, grid, dim3(256), 0, s, p);
    return rgd_launch_status(which == 0 ? "rgd_attn_bwd (prep)" : "rgd_attn_bwd (dq convert)", e);
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
    return rgd_launch_status("rgd_attn_bwd (merge)", rgd_launch(attn_bwd_merge_kernel<T, DPAD>, dim3(items, gy, nt), dim3(256), 0, s, p, nt));
}

template <typename T> int dispatch_bwd_merge(const AttnBwdParams& p, unsigned items, int nt, hipStream_t s) {
    if (p.D <= 32) return launch_bwd_merge<T, 32>(p, items, nt, s);
    if (p.D <= 64) return launch_bwd_merge<T, 64>(p, items, nt, s);
    if (p.D <= 96) return launch_bwd_merge<T, 96>(p, items, nt, s);
    return launch_bwd_merge<T, 128>(p, items, nt, s);
}

// Kernels that use more than 48 KB of dynamic LDS need hipFuncAttributeMaxDynamicSharedMemorySize before their first
// launch.  Called once per process from the library's set-up, for every instantiation of this element type, so no
// entry point touches function attributes afterwards (an entry point may run under stream capture, where such a
// call is not allowed).
template <typename T, int DPAD, int BIAS> const void* dq_dbias_kernel_ptr() {
    if constexpr (BIAS != BIAS_OFF) return reinterpret_cast<const void*>(attn_bwd_dq_kernel<T, DPAD, BIAS, true>);
    else return nullptr;
}
template <typename T, int DPAD, int BIAS> const void* fused_kernel_ptr() {
    if constexpr (DPAD <= 64) return reinterpret_cast<const void*>(attn_bwd_dkv_kernel<T, DPAD, BIAS, true>);
    else return nullptr;
}
template <int DPAD, int BIAS> constexpr size_t fused_kernel_lds() {
    if constexpr (DPAD <= 64) return DkvSmem<DPAD, dkv_nsub(DPAD, BIAS, true), true>::BYTES;
    else return 0;
}
template <typename T, int DPAD, int BIAS> int attn_configure_one() {
    struct K {
        const void* fn;
        size_t lds;
    };
    const K ks[] = {
        {reinterpret_cast<const void*>(attn_fwd_kernel<T, DPAD, BIAS>), AttnFwdSmem<DPAD>::BYTES},
        {reinterpret_cast<const void*>(attn_bwd_dq_kernel<T, DPAD, BIAS>), DqSmem<DPAD>::BYTES},
        {dq_dbias_kernel_ptr<T, DPAD, BIAS>(), DqSmem<DPAD>::BYTES},
        {reinterpret_cast<const void*>(attn_bwd_dkv_kernel<T, DPAD, BIAS>), DkvSmem<DPAD, dkv_nsub(DPAD, BIAS)>::BYTES},
        {fused_kernel_ptr<T, DPAD, BIAS>(), fused_kernel_lds<DPAD, BIAS>()},
    };
    for (const K& k : ks) {
        if (k.fn == nullptr || k.lds <= 48 * 1024) continue;
        if (hipFuncSetAttribute(k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)k.lds) != hipSuccess) {
            (void)hipGetLastError();
            rgd_set_error("rgd_init: cannot reserve %zu bytes of LDS for an attention kernel", k.lds);
            return RGD_ERR_LAUNCH;
        }
    }
    return RGD_OK;
}
template <typename T, int DPAD> int attn_configure_dpad() {
    int rc = attn_configure_one<T, DPAD, BIAS_OFF>();
    if (rc == RGD_OK) rc = attn_configure_one<T, DPAD, BIAS_SAME>();
    if (rc == RGD_OK) rc = attn_configure_one<T, DPAD, BIAS_F32>();
    return rc;
}
template <typename T> int attn_configure_all() {
    int rc = attn_configure_dpad<T, 32>();
    if (rc == RGD_OK) rc = attn_configure_dpad<T, 64>();
    if (rc == RGD_OK) rc = attn_configure_dpad<T, 96>();
    if (rc == RGD_OK) rc = attn_configure_dpad<T, 128>();
    return rc;
}
