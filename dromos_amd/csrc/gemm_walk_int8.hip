// The walk kernel on INT8 weights.
#include "gemm_walk.h"

namespace dro {
bool launch_walk_int8(const GemmArgs& a, int W, int* status, hipStream_t stream) { return walk::launch_format<LX_W_INT8>(a, W, status, stream); }
}  // namespace dro
