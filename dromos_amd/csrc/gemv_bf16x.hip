// The decode GEMV kernels of one weight format (a source per format, so they compile side by side).
#include "gemv_kernels.h"

namespace dro {

int gemv_launch_bf16x(GemvArgs& a, hipStream_t stream) { return launch_format<LX_W_BF16X>(a, "gemv_w_bf16x", stream); }

}  // namespace dro
