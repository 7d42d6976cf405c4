// k_gemv instantiations for CTHIP_F16 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvF16[] = {
    GEMV_SHAPES_F16(V)
};
extern const int kGemvF16Count = (int)(sizeof(kGemvF16) / sizeof(kGemvF16[0]));
}  // namespace cthip
