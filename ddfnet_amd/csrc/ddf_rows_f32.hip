// Row-register kernels, fp32 storage.
#include "ddf_rows_launch.h"

namespace ddf {
DDF_INSTANTIATE_ROWS(float)
}  // namespace ddf
