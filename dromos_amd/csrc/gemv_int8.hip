// The decode GEMV kernels of one weight format (a source per format, so they compile side by side).
#include "gemv_kernels.h"

namespace dro {

int gemv_launch_int8(GemvArgs& a, hipStream_t stream) { return launch_format<LX_W_INT8>(a, "gemv_w_int8", stream); }

}  // namespace dro
