// k_gemv instantiations for CTHIP_F16 weights (see gemv_kernels.h).
#include "gemv_kernels.h"

namespace cthip {
extern const GemvVariant kGemvF16[] = {
    V(CTHIP_F16, 16, 2), V(CTHIP_F16, 64, 1), V(CTHIP_F16, 64, 2), V(CTHIP_F16, 64, 3), V(CTHIP_F16, 64, 4), V(CTHIP_F16, 64, 6), V(CTHIP_F16, 64, 8), V(CTHIP_F16, 64, 12),
};
extern const int kGemvF16Count = (int)(sizeof(kGemvF16) / sizeof(kGemvF16[0]));
}  // namespace cthip
