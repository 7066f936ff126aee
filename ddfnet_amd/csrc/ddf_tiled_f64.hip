// Tiled DDF kernels instantiated for double.
#include "ddf_tiled_launch.h"

namespace ddf {
DDF_INSTANTIATE_TILED(double)
}  // namespace ddf
