// head_rows_kernel instantiations for f16_t rows
#include "rows_head_inst.h"
template int head_dispatch<f16_t>(const HeadConfig&, const HeadParams&, dim3, hipStream_t);
