// attention kernel instantiations for bf16_t with tile classes of a head-shared bias
#include "attn_cls_inst.h"
template int dispatch_fwd_cls<bf16_t>(const AttnFwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_cls<bf16_t, true>(const AttnBwdParams&, unsigned, hipStream_t);
template int dispatch_bwd_cls<bf16_t, false>(const AttnBwdParams&, unsigned, hipStream_t);
template int attn_configure_cls<bf16_t>();
