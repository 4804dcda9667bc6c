// The walk kernel on BF16 weights.
#include "gemm_walk.h"

namespace dro {
bool launch_walk_bf16(const GemmArgs& a, int W, int* status, hipStream_t stream) { return walk::launch_format<LX_W_BF16>(a, W, status, stream); }
}  // namespace dro
