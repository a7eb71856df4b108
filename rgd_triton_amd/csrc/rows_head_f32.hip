// head_rows_kernel instantiations for float rows
#include "rows_head_inst.h"
template int head_dispatch<float>(const HeadConfig&, const HeadParams&, dim3, hipStream_t);
