// Instantiates the attention kernels that read the tile classes of a head-shared bias (attn_classes.h) for one element
// type: head dims up to 64, bias in the tensor dtype or fp32.  Included by attn_cls_f16.hip and attn_cls_bf16.hip (units
// of their own so that they compile beside the ordinary instantiations).
#pragma once

#include "attn_fwd.h"
#include "attn_bwd.h"

template <typename T, int DPAD, int BIAS> int launch_fwd_cls(const AttnFwdParams& p, unsigned grid, hipStream_t s) {
    constexpr size_t lds = AttnFwdSmem<DPAD>::BYTES + CLS_LDS_BYTES;
    return rgd_launch_status("rgd_attn_fwd", rgd_launch(attn_fwd_kernel<T, DPAD, BIAS, true>, dim3(grid), dim3(ATTN_THREADS), lds, s, p));
}
template <typename T> int dispatch_fwd_cls(const AttnFwdParams& p, unsigned grid, hipStream_t s) {
    const bool f32 = p.bias_dtype == RGD_F32;
    if (p.D <= 32) return f32 ? launch_fwd_cls<T, 32, BIAS_F32>(p, grid, s) : launch_fwd_cls<T, 32, BIAS_SAME>(p, grid, s);
    if (p.D <= 64) return f32 ? launch_fwd_cls<T, 64, BIAS_F32>(p, grid, s) : launch_fwd_cls<T, 64, BIAS_SAME>(p, grid, s);
    return RGD_ERR_UNSUPPORTED;
}
template <typename T, int DPAD, int BIAS, bool DQ> int launch_bwd_cls(const AttnBwdParams& p, unsigned grid, hipStream_t s) {
    constexpr size_t lds = DQ ? DqSmem<DPAD>::BYTES + CLS_LDS_BYTES : DkvSmem<DPAD, dkv_nsub(DPAD, BIAS_OFF)>::BYTES;
    auto kern = DQ ? attn_bwd_dq_kernel<T, DPAD, BIAS, false, true> : attn_bwd_dkv_kernel<T, DPAD, BIAS, false, true>;
    return rgd_launch_status("rgd_attn_bwd", rgd_launch(kern, dim3(grid), dim3(BWD_THREADS), lds, s, p));
}
template <typename T, bool DQ> int dispatch_bwd_cls(const AttnBwdParams& p, unsigned grid, hipStream_t s) {
    const bool f32 = p.bias_dtype == RGD_F32;
    if (p.D <= 32) return f32 ? launch_bwd_cls<T, 32, BIAS_F32, DQ>(p, grid, s) : launch_bwd_cls<T, 32, BIAS_SAME, DQ>(p, grid, s);
    if (p.D <= 64) return f32 ? launch_bwd_cls<T, 64, BIAS_F32, DQ>(p, grid, s) : launch_bwd_cls<T, 64, BIAS_SAME, DQ>(p, grid, s);
    return RGD_ERR_UNSUPPORTED;
}


// LDS size attribute of every kernel above (see attn_configure_all)
template <typename T, int DPAD, int BIAS> int attn_configure_cls_one() {
    struct K {
        const void* fn;
        size_t lds;
    };
    const K ks[] = {
        {reinterpret_cast<const void*>(attn_fwd_kernel<T, DPAD, BIAS, true>), AttnFwdSmem<DPAD>::BYTES + CLS_LDS_BYTES},
        {reinterpret_cast<const void*>(attn_bwd_dq_kernel<T, DPAD, BIAS, false, true>), DqSmem<DPAD>::BYTES + CLS_LDS_BYTES},
        {reinterpret_cast<const void*>(attn_bwd_dkv_kernel<T, DPAD, BIAS, false, true>), DkvSmem<DPAD, dkv_nsub(DPAD, BIAS_OFF)>::BYTES},
    };
    for (const K& k : ks) {
        if (k.lds <= 48 * 1024) continue;
        if (hipFuncSetAttribute(k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)k.lds) != hipSuccess) {
            (void)hipGetLastError();
            rgd_set_error("rgd_init: cannot reserve %zu bytes of LDS for an attention kernel", k.lds);
            return RGD_ERR_LAUNCH;
        }
    }
    return RGD_OK;
}
template <typename T> int attn_configure_cls() {
    int rc = attn_configure_cls_one<T, 32, BIAS_SAME>();
    if (rc == RGD_OK) rc = attn_configure_cls_one<T, 32, BIAS_F32>();
    if (rc == RGD_OK) rc = attn_configure_cls_one<T, 64, BIAS_SAME>();
    if (rc == RGD_OK) rc = attn_configure_cls_one<T, 64, BIAS_F32>();
    return rc;
}
