// Tiled DDF kernels instantiated for __half.
#include "ddf_tiled_launch.h"

namespace ddf {
DDF_INSTANTIATE_TILED(__half)
}  // namespace ddf
