// placeholder: tiled family not built yet
#include "ddf_common.h"
namespace ddf {
bool tiled_forward_supported(const Problem &, int) { return false; }
bool tiled_backward_supported(const Problem &, int) { return false; }
size_t tiled_backward_workspace(const Problem &, int, unsigned) { return 0; }
template <typename T>
hipError_t tiled_forward(const Problem &, const T *, const T *, const T *, T *, hipStream_t) { return hipErrorNotSupported; }
template <typename T>
hipError_t tiled_backward(const Problem &, const T *, const T *, const T *, const T *, T *, T *, T *, void *, unsigned, hipStream_t) { return hipErrorNotSupported; }
#define INST(T) \
 template hipError_t tiled_forward<T>(const Problem &, const T *, const T *, const T *, T *, hipStream_t); \
 template hipError_t tiled_backward<T>(const Problem &, const T *, const T *, const T *, const T *, T *, T *, T *, void *, unsigned, hipStream_t);
INST(__half) INST(float) INST(double)
}
