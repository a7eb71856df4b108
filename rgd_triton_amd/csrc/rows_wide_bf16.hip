// wide_rows_kernel instantiations for bf16_t rows
#include "rows_wide_inst.h"
template int wide_dispatch<bf16_t>(const WideConfig&, const WideParams&, dim3, size_t, hipStream_t);
