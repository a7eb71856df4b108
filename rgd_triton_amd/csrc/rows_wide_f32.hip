// wide_rows_kernel instantiations for float rows
#include "rows_wide_inst.h"
template int wide_dispatch<float>(const WideConfig&, const WideParams&, dim3, size_t, hipStream_t);
