// attention kernel instantiations for f16_t with tile classes of a head-shared bias
#include "attn_cls_inst.h"
template int dispatch_fwd_cls<f16_t>(const AttnFwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_cls<f16_t, true>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_cls<f16_t, false>(const AttnBwdParams&, unsigned, hipStream_t);
template int attn_configure_cls<f16_t>();
