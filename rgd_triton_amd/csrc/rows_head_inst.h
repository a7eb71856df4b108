// Instantiates head_rows_kernel for one element type and dispatches a run-time configuration to it.
#pragma once

#include "rows_head.h"

template <typename T, typename TP, int MODE, int G, int NV, bool VECTOR>
static int head_launch_one(const HeadParams& p, bool compact, dim3 grid, hipStream_t s) {
    constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 2;
    constexpr int U = head_unroll(MODE, NV);
    // rows that fill their lane group exactly (the power-of-two head dims) skip every range mask
    if (VECTOR && p.D == G * NV * VEC) {
        if (compact)
            return rgd_launch_status("head rows", rgd_launch(head_rows_kernel<T, TP, MODE, G, NV, VEC, VECTOR, VECTOR, U, VECTOR>, grid, dim3(256), 0, s, p));
        return rgd_launch_status("head rows", rgd_launch(head_rows_kernel<T, TP, MODE, G, NV, VEC, VECTOR, VECTOR, U>, grid, dim3(256), 0, s, p));
    }
    return rgd_launch_status("head rows", rgd_launch(head_rows_kernel<T, TP, MODE, G, NV, VEC, VECTOR, false, U>, grid, dim3(256), 0, s, p));
}

template <typename T, typename TP, int MODE, bool VECTOR>
static int head_dispatch_shape(const HeadConfig& c, const HeadParams& p, dim3 grid, hipStream_t s) {
#define HEAD_CASE(g, nv) \
    if (c.G == g && c.NV == nv) return head_launch_one<T, TP, MODE, g, nv, VECTOR>(p, c.compact, grid, s);
    HEAD_CASE(4, 1)
    HEAD_CASE(8, 1)
    HEAD_CASE(16, 1)
    HEAD_CASE(32, 1)
    HEAD_CASE(64, 1)
    HEAD_CASE(64, 2)
#undef HEAD_CASE
    rgd_set_error("head rows: no kernel for G=%d NV=%d", c.G, c.NV);
    return RGD_ERR_UNSUPPORTED;
}

template <typename T, int MODE> static int head_dispatch_mode(const HeadConfig& c, const HeadParams& p, dim3 grid, hipStream_t s) {
    constexpr bool ROPE = MODE == HEAD_ROPE || MODE == HEAD_LNROPE_FWD || MODE == HEAD_LNROPE_BWD;
    if constexpr (ROPE && sizeof(T) == 2) {
        if (c.table_f32)
            return c.vector ? head_dispatch_shape<T, float, MODE, true>(c, p, grid, s)
                            : head_dispatch_shape<T, float, MODE, false>(c, p, grid, s);
    }
    return c.vector ? head_dispatch_shape<T, T, MODE, true>(c, p, grid, s)
                    : head_dispatch_shape<T, T, MODE, false>(c, p, grid, s);
}

template <typename T> int head_dispatch(const HeadConfig& c, const HeadParams& p, dim3 grid, hipStream_t s) {
#define HEAD_MODE(M_) \
    if (c.mode == M_) return head_dispatch_mode<T, M_>(c, p, grid, s);
    HEAD_MODE(HEAD_LN_FWD)
    HEAD_MODE(HEAD_LN_BWD)
    HEAD_MODE(HEAD_ROPE)
    HEAD_MODE(HEAD_LNROPE_FWD)
    HEAD_MODE(HEAD_LNROPE_BWD)
#undef HEAD_MODE
    rgd_set_error("head rows: bad mode %d", c.mode);
    return RGD_ERR_INVALID;
}
