// Instantiates wide_rows_kernel for one element type and dispatches a run-time configuration to it.
// Included by rows_wide_f32.hip / rows_wide_f16.hip / rows_wide_bf16.hip so the three element
// types compile in parallel.
#pragma once

#include "rows_wide.h"

template <typename T, int OP, bool BWD, int G, int NV, bool VECTOR, int WPR>
static int wide_launch_one(const WideParams& p, dim3 grid, size_t lds, hipStream_t s) {
    constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 2;
    constexpr int U = wide_unroll(BWD, NV, VEC);
    constexpr int NW = wide_waves(OP, BWD);
    // the host never selects more elements per lane than this (they would not stay in registers)
    if constexpr (NV * VEC <= ((OP == WIDE_RMS && (BWD || !RGD_WIDE_RMS_FWD_64)) ? 32 : 64)) {
        return rgd_launch_status("wide rows", rgd_launch(wide_rows_kernel<T, OP, BWD, G, NV, VEC, VECTOR, U, NW, WPR>, grid,
                                                         dim3(NW * 64), lds, s, p));
    }
    rgd_set_error("wide rows: %d elements per lane were not compiled", NV * VEC);
    return RGD_ERR_UNSUPPORTED;
}

template <typename T, int OP, bool BWD, bool VECTOR>
static int wide_dispatch_shape(const WideConfig& c, const WideParams& p, dim3 grid, size_t lds, hipStream_t s) {
#define WIDE_CASE(g, nv) \
    if (c.WPR == 1 && c.G == g && c.NV == nv) return wide_launch_one<T, OP, BWD, g, nv, VECTOR, 1>(p, grid, lds, s);
#define WIDE_CASE4(nv) \
    if (c.WPR == 4 && c.G == 64 && c.NV == nv) return wide_launch_one<T, OP, BWD, 64, nv, VECTOR, 4>(p, grid, lds, s);
    WIDE_CASE(4, 1)
    WIDE_CASE(8, 1)
    WIDE_CASE(16, 1)
    WIDE_CASE(32, 1)
    WIDE_CASE(64, 1)
    WIDE_CASE(64, 2)
    WIDE_CASE(64, 3)
    WIDE_CASE(64, 4)
    WIDE_CASE(64, 6)
    WIDE_CASE(64, 8)
    WIDE_CASE(64, 12)
    WIDE_CASE(64, 16)
    WIDE_CASE4(1)
    WIDE_CASE4(2)
    WIDE_CASE4(3)
    WIDE_CASE4(4)
    WIDE_CASE4(6)
    WIDE_CASE4(8)
    WIDE_CASE4(12)
    WIDE_CASE4(16)
#undef WIDE_CASE
#undef WIDE_CASE4
    rgd_set_error("wide rows: no kernel for G=%d NV=%d WPR=%d", c.G, c.NV, c.WPR);
    return RGD_ERR_UNSUPPORTED;
}

template <typename T, int OP, bool BWD, bool VECTOR>
static int wide_launch_stream(const WideParams& p, dim3 grid, hipStream_t s) {
    constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 2;
    constexpr int NKW = (OP == WIDE_RMS && BWD) ? wide_stream_nkw(VEC) : 0;
    return rgd_launch_status("wide rows (streaming)", rgd_launch(wide_stream_kernel<T, OP, BWD, VEC, VECTOR, NKW>, grid, dim3(256), 0, s, p));
}

template <typename T>
int wide_dispatch(const WideConfig& c, const WideParams& p, dim3 grid, size_t lds, hipStream_t s) {
#define WIDE_STREAM(OP_, BWD_)                                                            \
    if (c.stream && c.op == OP_ && c.bwd == BWD_)                                         \
        return c.vector ? wide_launch_stream<T, OP_, BWD_, true>(p, grid, s)              \
                        : wide_launch_stream<T, OP_, BWD_, false>(p, grid, s);
    WIDE_STREAM(WIDE_RMS, false)
    WIDE_STREAM(WIDE_RMS, true)
    WIDE_STREAM(WIDE_L2, false)
    WIDE_STREAM(WIDE_L2, true)
#undef WIDE_STREAM
#define WIDE_OP(OP_, BWD_)                                                                      \
    if (c.op == OP_ && c.bwd == BWD_)                                                           \
        return c.vector ? wide_dispatch_shape<T, OP_, BWD_, true>(c, p, grid, lds, s)           \
                        : wide_dispatch_shape<T, OP_, BWD_, false>(c, p, grid, lds, s);
    WIDE_OP(WIDE_RMS, false)
    WIDE_OP(WIDE_RMS, true)
    WIDE_OP(WIDE_L2, false)
    WIDE_OP(WIDE_L2, true)
#undef WIDE_OP
    rgd_set_error("wide rows: bad op %d", c.op);
    return RGD_ERR_INVALID;
}
