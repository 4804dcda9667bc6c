// The decode GEMV kernels of one weight format (a source per format, so they compile side by side).
#include "gemv_kernels.h"

namespace dro {

// The encoded product promises the bf16 product's bits, so it takes its K split from the bf16 kernel's entry in the
// variant table: a split tuned or forced for one is the other's too.
int gemv_launch_bf16x(GemvArgs& a, hipStream_t stream) { return launch_format<LX_W_BF16X>(a, "gemv_w_bf16", stream); }

}  // namespace dro
