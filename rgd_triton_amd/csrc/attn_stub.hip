// temporary: attention entry points until the MFMA kernels land
#include "common.h"
extern "C" {
int64_t rgd_attn_seqlen_q_rounded(int64_t Tq) { return (Tq + 63) / 64 * 64; }
int rgd_attn_fwd(int64_t, int64_t, int64_t, int64_t, int64_t, const rgd_tensor4*, const rgd_tensor4*, const rgd_tensor4*,
                 const rgd_tensor4*, int, int, const rgd_tensor4*, float*, int, int, float, void*) {
    rgd_set_error("rgd_attn_fwd: not built");
    return RGD_ERR_UNSUPPORTED;
}
size_t rgd_attn_bwd_workspace(int64_t B, int64_t H, int64_t Tq, int64_t, int64_t) {
    return (size_t)(B * H * rgd_attn_seqlen_q_rounded(Tq)) * sizeof(float);
}
int rgd_attn_bwd(int64_t, int64_t, int64_t, int64_t, int64_t, const rgd_tensor4*, const rgd_tensor4*, const rgd_tensor4*,
                 const rgd_tensor4*, const rgd_tensor4*, const float*, const rgd_tensor4*, int, int, const rgd_tensor4*,
                 const rgd_tensor4*, const rgd_tensor4*, int, int, float, void*, size_t, void*) {
    rgd_set_error("rgd_attn_bwd: not built");
    return RGD_ERR_UNSUPPORTED;
}
}
