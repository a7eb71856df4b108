// head_rows_kernel instantiations for bf16_t rows
#include "rows_head_inst.h"
template int head_dispatch<bf16_t>(const HeadConfig&, const HeadParams&, dim3, hipStream_t);
