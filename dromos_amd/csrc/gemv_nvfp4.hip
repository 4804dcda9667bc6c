// The decode GEMV kernels of one weight format (a source per format, so they compile side by side).
#include "gemv_kernels.h"

namespace dro {

int gemv_launch_nvfp4(GemvArgs& a, hipStream_t stream) { return launch_format<LX_W_NVFP4>(a, "gemv_w_nvfp4", stream); }

}  // namespace dro
