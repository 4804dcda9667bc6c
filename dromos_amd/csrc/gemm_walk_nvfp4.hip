// The walk kernel on NVFP4 weights.
#include "gemm_walk.h"

namespace dro {
bool launch_walk_nvfp4(const GemmArgs& a, int W, int* status, hipStream_t stream) { return walk::launch_format<LX_W_NVFP4>(a, W, status, stream); }
}  // namespace dro
