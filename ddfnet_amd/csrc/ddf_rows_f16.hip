// Row-register kernels, fp16 storage (fp32 accumulation).
#include "ddf_rows_launch.h"

namespace ddf {
DDF_INSTANTIATE_ROWS(__half)
}  // namespace ddf
