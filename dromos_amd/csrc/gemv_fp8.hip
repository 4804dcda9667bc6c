// The decode GEMV kernels of one weight format (a source per format, so they compile side by side).
#include "gemv_kernels.h"

namespace dro {

int gemv_launch_fp8(GemvArgs& a, hipStream_t stream) { return launch_format<LX_W_FP8>(a, "gemv_w_fp8", stream); }

}  // namespace dro
