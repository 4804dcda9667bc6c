// The walk kernel on FP8 weights.
#include "gemm_walk.h"

namespace dro {
bool launch_walk_fp8(const GemmArgs& a, int W, int* status, hipStream_t stream) { return walk::launch_format<LX_W_FP8>(a, W, status, stream); }
}  // namespace dro
