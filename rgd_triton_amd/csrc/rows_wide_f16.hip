// wide_rows_kernel instantiations for f16_t rows
#include "rows_wide_inst.h"
template int wide_dispatch<f16_t>(const WideConfig&, const WideParams&, dim3, size_t, hipStream_t);
