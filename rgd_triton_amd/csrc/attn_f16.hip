// attention kernel instantiations for f16_t
#include "attn_inst.h"
template int dispatch_fwd<f16_t>(const AttnFwdParams&, unsigned, hipStream_t);
template int dispatch_fwd_merge<f16_t>(const AttnFwdParams&, unsigned, hipStream_t);
template int dispatch_bwd<f16_t, true>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd<f16_t, false>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_merge<f16_t>(const AttnBwdParams&, unsigned, int, hipStream_t);
template int attn_configure_all<f16_t>();
template int dispatch_bwd_fused<f16_t>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_fused_aux<f16_t>(const AttnBwdParams&, int, hipStream_t);
