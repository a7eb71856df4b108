// attention kernel instantiations for bf16_t
#include "attn_inst.h"
template int dispatch_fwd<bf16_t>(const AttnFwdParams&, unsigned, hipStream_t);
template int dispatch_fwd_merge<bf16_t>(const AttnFwdParams&, unsigned, hipStream_t);
template int dispatch_bwd<bf16_t, true>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd<bf16_t, false>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_merge<bf16_t>(const AttnBwdParams&, unsigned, int, hipStream_t);
template int attn_configure_all<bf16_t>();
template int dispatch_bwd_fused<bf16_t>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_fused_aux<bf16_t>(const AttnBwdParams&, int, hipStream_t);
