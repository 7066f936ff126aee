// Tiled DDF kernels instantiated for float.
#include "ddf_tiled_launch.h"

namespace ddf {
DDF_INSTANTIATE_TILED(float)
}  // namespace ddf
